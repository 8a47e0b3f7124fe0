// Dense linear layers: C[M,N] = alpha * A[M,K] * B[N,K]^T + beta * C, all FP16
// row-major, FP32 accumulation.
//
// Both operands are contiguous along K, which is what the CDNA4 matrix core
// wants: v_mfma_f32_32x32x16_f16 takes, per lane, eight consecutive K values
// of one row of each operand. The kernels:
//
//   gemm_tile<BM,BN,WM,WN>  workgroup tile BM x BN over WM x WN waves, K in
//                           slabs of 64 or 32 staged through LDS (double-buffered,
//                           16-byte slots XOR-swizzled so that the 32 rows a
//                           ds_read_b128 touches fall in distinct banks). The
//                           weight rows are the MFMA's A operand and the
//                           activation rows its B operand, so a lane ends up
//                           with four CONSECUTIVE output columns of one output
//                           row: 8-byte stores. Every tile shape adds the K
//                           slabs in the same order, so all of them produce
//                           the same bits for the same element.
//   gemm_dma                the 256x256 tile for large problems: slabs copied
//                           from global memory straight into LDS (no staging
//                           registers), four LDS stages, same K order.
//   gemm_skinny<kMT>        2 <= M <= 64: the weights go from global memory
//                           straight into 16x16x32 MFMA operands, K split
//                           over the eight waves of a workgroup; bound by the
//                           weight bytes.
//   gemm_skinny_lines<kMT>  the same for FP16 weights and K % 64 == 0: both
//                           operands come by whole cache lines through each
//                           wave's own LDS ring (same bits).
//   gemv_row<kSplit>        M == 1 (a decode step): one to four waves per
//                           output column stream that weight row once with
//                           non-temporal 16-byte loads.
//   gemv_rows<kSplit, kR>   M == 1 over few long weight rows: kR output
//                           columns per wave, summed in gemv_row's order.
//   gemm_naive              K not a multiple of 8, or pointers off 16 bytes.
#include "mfma_dma.hpp"
#include "row_math.hpp"
#include "wonly.hpp"

namespace vv {
namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float finish(float acc, float alpha, float beta, h16 old) {
    return alpha * acc + beta * (float)old;
}

// A wave's TN x TM accumulator tiles to C. Result register 4g + r of lane l holds
// column n0 + 8g + 4(l / 32) + r of row m0 + l % 32 of its 32x32 tile.
template <int TM, int TN>
__device__ __forceinline__ void store_tile(const f32x16 (&acc)[TN][TM], h16* __restrict__ C, int M,
                                           int N, int m0, int n0, int frow, int fhalf, float alpha,
                                           float beta, int vec_store) {
#pragma unroll
    for (int b = 0; b < TM; ++b) {
        const int m = m0 + b * 32 + frow;
        if (m >= M) continue;
        h16* crow = C + (size_t)m * N;
#pragma unroll
        for (int a = 0; a < TN; ++a) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int n = n0 + a * 32 + 8 * g + 4 * fhalf;
                if (n >= N) continue;
                if (vec_store && n + 3 < N) {
                    typedef h16 h16x4 __attribute__((ext_vector_type(4)));
                    h16x4 old = {0, 0, 0, 0};
                    if (beta != 0.0f) old = *reinterpret_cast<const h16x4*>(crow + n);
                    h16x4 o;
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        o[r] = to_half(finish(acc[a][b][4 * g + r], alpha, beta, old[r]));
                    *reinterpret_cast<h16x4*>(crow + n) = o;
                } else {
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (n + r < N) {
                            const h16 old = beta != 0.0f ? crow[n + r] : (h16)0.0f;
                            crow[n + r] = to_half(finish(acc[a][b][4 * g + r], alpha, beta, old));
                        }
                }
            }
        }
    }
}

struct F16Op {
    typedef f32x16 Acc;
    static __device__ __forceinline__ Acc mfma(u32x4 w, u32x4 x, Acc c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h16x8, w),
                                                      __builtin_bit_cast(h16x8, x), c, 0, 0, 0);
    }
    typedef f32x4 Acc16;
    static __device__ __forceinline__ Acc16 mfma16(u32x4 w, u32x4 x, Acc16 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h16x8, w),
                                                      __builtin_bit_cast(h16x8, x), c, 0, 0, 0);
    }
};

// A wave's 4 x TM accumulator tiles of 16 x 16 (mfma_dma64) to C: register r of lane l holds column
// n0 + 16 a + 4 (l / 16) + r of row m0 + 16 b + l % 16 of acc[a][b]. C's rows are ldc halves apart (the launch
// may cover a range of C's columns).
template <int TM>
__device__ __forceinline__ void store_tile16(const f32x4 (&acc)[4][TM], h16* __restrict__ C, int M, int N, int ldc,
                                             int m0, int n0, int lane, float alpha, float beta, int vec_store) {
    typedef h16 h16x4 __attribute__((ext_vector_type(4)));
#pragma unroll
    for (int b = 0; b < TM; ++b) {
        const int m = m0 + b * 16 + (lane & 15);
        if (m >= M) continue;
        h16* crow = C + (size_t)m * ldc;
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const int n = n0 + a * 16 + 4 * (lane >> 4);
            if (n >= N) continue;
            if (vec_store && n + 3 < N) {
                h16x4 old = {0, 0, 0, 0};
                if (beta != 0.0f) old = *reinterpret_cast<const h16x4*>(crow + n);
                h16x4 o;
#pragma unroll
                for (int r = 0; r < 4; ++r) o[r] = to_half(finish(acc[a][b][r], alpha, beta, old[r]));
                *reinterpret_cast<h16x4*>(crow + n) = o;
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (n + r < N) {
                        const h16 old = beta != 0.0f ? crow[n + r] : (h16)0.0f;
                        crow[n + r] = to_half(finish(acc[a][b][r], alpha, beta, old));
                    }
            }
        }
    }
}

template <int BM, int BN, int WM, int WN, int kSlab, bool kFull, int kAhead>
__global__ __launch_bounds__(WM * WN * kWave) void gemm_tile(
    const h16* __restrict__ A, const h16* __restrict__ B, h16* __restrict__ C, int M, int N,
    int K, float alpha, float beta, int vec_store) {
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    auto epilogue = [=](const f32x16 (&acc)[TN][TM], int m0, int n0, int frow, int fhalf) {
        store_tile<TM, TN>(acc, C, M, N, m0, n0, frow, fhalf, alpha, beta, vec_store);
    };
    mfma_tile<F16Op, BM, BN, WM, WN, kSlab / 8, kFull, kAhead>(A, B, M, N, K / 8, epilogue);
}

// The same tile loop with the weight rows dequantised on their way in (wonly.hpp): the K order of gemm_tile, so
// the bits of dequantising into FP16 first and running gemm_tile on that.
template <int kFmt>
struct WoRows {
    static constexpr bool kPlain = false;
    WoSource src;
    const float* book;
    int K;
    __device__ __forceinline__ u32x4 load(int row, int slot) const { return wo_slot<kFmt>(src, book, (size_t)row, K, slot); }
};

template <int BM, int BN, int WM, int WN, int kSlab, bool kFull, int kFmt>
__global__ __launch_bounds__(WM * WN * kWave) void gemm_tile_wo(
    const h16* __restrict__ A, WoSource B, h16* __restrict__ C, int M, int N, int K, int vec_store) {
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    __shared__ float book[16];
    if constexpr (kFmt == kWoNf4) {
        if (threadIdx.x < 16) book[threadIdx.x] = kNf4Book[threadIdx.x];
        __syncthreads();
    }
    auto epilogue = [=](const f32x16 (&acc)[TN][TM], int m0, int n0, int frow, int fhalf) {
        store_tile<TM, TN>(acc, C, M, N, m0, n0, frow, fhalf, 1.0f, 0.0f, vec_store);
    };
    const WoRows<kFmt> rows = {B, book, K};
    mfma_tile<F16Op, BM, BN, WM, WN, kSlab / 8, kFull, 1>(A, nullptr, M, N, K / 8, epilogue, rows);
}

// The 256x256 tile with the slabs copied from global memory straight into LDS
// (mfma_dma.hpp). Needs K % 32 == 0.
__global__ __launch_bounds__(kDmaWaves * kWave) void gemm_dma(
    const h16* __restrict__ A, const h16* __restrict__ B, h16* __restrict__ C, int M, int N,
    int K, float alpha, float beta, int vec_store) {
    auto epilogue = [=](const f32x16 (&acc)[2][4], int m0, int n0, int frow, int fhalf) {
        store_tile<4, 2>(acc, C, M, N, m0, n0, frow, fhalf, alpha, beta, vec_store);
    };
    mfma_dma<F16Op>(A, B, M, N, K * 2, epilogue);
}

// The 256x256 or 128x128 tile fed in slabs of 64 halves (whole cache lines per row; mfma_dma.hpp). Needs
// K % 64 == 0.
template <int kTile, int kStages>
__global__ __launch_bounds__(Dma64Shape<kTile>::kWaves * kWave, 2) void gemm_dma64(
    const h16* __restrict__ A, const h16* __restrict__ B, h16* __restrict__ C, int M, int N,
    int K, int ldc, float alpha, float beta, int vec_store) {
    constexpr int TM = Dma64Shape<kTile>::TM;
    auto epilogue = [=](const f32x4 (&acc)[4][TM], int m0, int n0, int lane) {
        store_tile16<TM>(acc, C, M, N, ldc, m0, n0, lane, alpha, beta, vec_store);
    };
    mfma_dma64<F16Op, kTile, false, kStages>(A, B, M, N, K * 2, epilogue);
}

// The projection epilogue of a rotary attention layer in the GEMM's store: C = rope(fp16(A W^T) + bias)
// for heads of 128 columns. The wave's two N tiles are 64 columns apart (kPairN), so register 4g + r of
// acc[0] and of acc[1] are columns n and n + 64 of one head: the rotate-half pair. Every step rounds where
// the separate launches round - the product to FP16 (the GEMM's store), the biased value to FP16 (the bias
// add's store), then the unfused rotation of the rope kernels on cos/sin read from a table that holds
// their sincosf values - so the result equals GEMM, then bias + RoPE, bit for bit.
template <int TM>
__device__ __forceinline__ void store_tile_rope(const f32x16 (&acc)[2][TM], h16* __restrict__ C,
                                                const h16* __restrict__ bias, const float2* __restrict__ table,
                                                int M, int N, int m0, int n0, int frow, int fhalf, float alpha,
                                                float beta) {
    typedef h16 h16x4 __attribute__((ext_vector_type(4)));
    if (n0 >= N) return;                         // whole heads: the wave's 64 + 64 columns are all in or all out
    const int pair0 = n0 & 127;                  // 0 or 32: the first rotation pair of tile 0
#pragma unroll
    for (int b = 0; b < TM; ++b) {
        const int m = m0 + b * 32 + frow;
        if (m >= M) continue;
        h16* crow = C + (size_t)m * N;
        const float2* trow = table + (size_t)m * 64;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int col = 8 * g + 4 * fhalf;
            const int n = n0 + col;
            h16x4 lo, hi;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                lo[r] = to_half(finish(acc[0][b][4 * g + r], alpha, beta, (h16)0.0f));
                hi[r] = to_half(finish(acc[1][b][4 * g + r], alpha, beta, (h16)0.0f));
            }
            if (bias) {
                const h16x4 blo = *reinterpret_cast<const h16x4*>(bias + n);
                const h16x4 bhi = *reinterpret_cast<const h16x4*>(bias + n + 64);
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    lo[r] = to_half((float)lo[r] + (float)blo[r]);
                    hi[r] = to_half((float)hi[r] + (float)bhi[r]);
                }
            }
            const float4 cs01 = *reinterpret_cast<const float4*>(trow + pair0 + col);
            const float4 cs23 = *reinterpret_cast<const float4*>(trow + pair0 + col + 2);
            const float cv[4] = {cs01.x, cs01.z, cs23.x, cs23.z};
            const float sv[4] = {cs01.y, cs01.w, cs23.y, cs23.w};
            h16x4 olo, ohi;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const Pair p = rotate((float)lo[r], (float)hi[r], cv[r], sv[r]);
                olo[r] = to_half(p.lo);
                ohi[r] = to_half(p.hi);
            }
            *reinterpret_cast<h16x4*>(crow + n) = olo;
            *reinterpret_cast<h16x4*>(crow + n + 64) = ohi;
        }
    }
}

// The same store for mfma_dma64's 16 x 16 tiles (kPairN: tiles a and a + 2 are 64 columns apart, tile a at
// column 16 (a % 2) + 64 (a / 2) of the wave's head half): register r of acc[a][b] and of acc[a + 2][b] are the
// rotate-half pair.
template <int TM>
__device__ __forceinline__ void store_tile16_rope(const f32x4 (&acc)[4][TM], h16* __restrict__ C,
                                                  const h16* __restrict__ bias, const float2* __restrict__ table,
                                                  int M, int N, int ldc, int m0, int n0, int lane, float alpha,
                                                  float beta) {
    typedef h16 h16x4 __attribute__((ext_vector_type(4)));
    if (n0 >= N) return;                         // whole heads: the wave's 32 + 32 columns are all in or all out
    const int pair0 = n0 & 127;                  // 0 or 32: the first rotation pair of tile 0
#pragma unroll
    for (int b = 0; b < TM; ++b) {
        const int m = m0 + b * 16 + (lane & 15);
        if (m >= M) continue;
        h16* crow = C + (size_t)m * ldc;
        const float2* trow = table + (size_t)m * 64;
#pragma unroll
        for (int a = 0; a < 2; ++a) {
            const int col = 16 * a + 4 * (lane >> 4);
            const int n = n0 + col;
            h16x4 lo, hi;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                lo[r] = to_half(finish(acc[a][b][r], alpha, beta, (h16)0.0f));
                hi[r] = to_half(finish(acc[a + 2][b][r], alpha, beta, (h16)0.0f));
            }
            if (bias) {
                const h16x4 blo = *reinterpret_cast<const h16x4*>(bias + n);
                const h16x4 bhi = *reinterpret_cast<const h16x4*>(bias + n + 64);
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    lo[r] = to_half((float)lo[r] + (float)blo[r]);
                    hi[r] = to_half((float)hi[r] + (float)bhi[r]);
                }
            }
            const float4 cs01 = *reinterpret_cast<const float4*>(trow + pair0 + col);
            const float4 cs23 = *reinterpret_cast<const float4*>(trow + pair0 + col + 2);
            const float cv[4] = {cs01.x, cs01.z, cs23.x, cs23.z};
            const float sv[4] = {cs01.y, cs01.w, cs23.y, cs23.w};
            h16x4 olo, ohi;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const Pair p = rotate((float)lo[r], (float)hi[r], cv[r], sv[r]);
                olo[r] = to_half(p.lo);
                ohi[r] = to_half(p.hi);
            }
            *reinterpret_cast<h16x4*>(crow + n) = olo;
            *reinterpret_cast<h16x4*>(crow + n + 64) = ohi;
        }
    }
}

template <int BM, int BN, int WM, int WN, int kSlab, bool kFull, int kAhead>
__global__ __launch_bounds__(WM * WN * kWave) void gemm_tile_rope(
    const h16* __restrict__ A, const h16* __restrict__ B, const h16* __restrict__ bias,
    const float2* __restrict__ table, h16* __restrict__ C, int M, int N, int K, float alpha, float beta) {
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    auto epilogue = [=](const f32x16 (&acc)[TN][TM], int m0, int n0, int frow, int fhalf) {
        store_tile_rope<TM>(acc, C, bias, table, M, N, m0, n0, frow, fhalf, alpha, beta);
    };
    mfma_tile<F16Op, BM, BN, WM, WN, kSlab / 8, kFull, kAhead, decltype(epilogue), PlainRows, true>(
        A, B, M, N, K / 8, epilogue);
}

__global__ __launch_bounds__(kDmaWaves * kWave) void gemm_dma_rope(
    const h16* __restrict__ A, const h16* __restrict__ B, const h16* __restrict__ bias,
    const float2* __restrict__ table, h16* __restrict__ C, int M, int N, int K, float alpha, float beta) {
    auto epilogue = [=](const f32x16 (&acc)[2][4], int m0, int n0, int frow, int fhalf) {
        store_tile_rope<4>(acc, C, bias, table, M, N, m0, n0, frow, fhalf, alpha, beta);
    };
    mfma_dma<F16Op, true>(A, B, M, N, K * 2, epilogue);
}

template <int kTile, int kStages>
__global__ __launch_bounds__(Dma64Shape<kTile>::kWaves * kWave, 2) void gemm_dma64_rope(
    const h16* __restrict__ A, const h16* __restrict__ B, const h16* __restrict__ bias,
    const float2* __restrict__ table, h16* __restrict__ C, int M, int N, int K, int ldc, float alpha, float beta) {
    constexpr int TM = Dma64Shape<kTile>::TM;
    auto epilogue = [=](const f32x4 (&acc)[4][TM], int m0, int n0, int lane) {
        store_tile16_rope<TM>(acc, C, bias, table, M, N, ldc, m0, n0, lane, alpha, beta);
    };
    mfma_dma64<F16Op, kTile, true, kStages>(A, B, M, N, K * 2, epilogue);
}

// The q, k and v projections of a chunk of rows in one grid (mfma_dma64_qkv): tile (tile_m, head) holds 128 rows
// of one q or k head - bias and RoPE in the store, as gemm_dma64_rope - and of v's columns 16 head .. + 15 (bias
// in the store). k and v rows go to plain [rows, n_kv_heads * 128] buffers and / or into an FP16 KV cache at
// positions first .. first + M - 1 (contiguous, or through a table of 64-position pages), so neither the bias
// add nor the append needs a launch of its own. Every step rounds where the separate launches round.
struct QkvArgs {
    const h16 *x, *wq, *wk, *wv, *bq, *bk, *bv;
    const float2* table;
    h16 *q, *k, *v, *k_cache, *v_cache;
    const int* page_table;
    const int* d_pos;
    int pos, M, K, n_q_heads, n_kv_heads;
};

template <int kStages>
__global__ __launch_bounds__(QkvShape<kStages>::kWaves * kWave, 2) void gemm_dma64_qkv(const QkvArgs g) {
    typedef h16 h16x4 __attribute__((ext_vector_type(4)));
    // Workgroup i runs on XCD i % 8 as its (i / 8)-th: an XCD takes eight heads (XCD % 4) and every other row
    // tile (XCD / 4), eight row tiles at a time, so the 64 workgroups it runs together share 8 + 8 operand tiles.
    const int xcd = (int)blockIdx.x & 7, nth = (int)blockIdx.x >> 3;
    const int n_heads = g.n_q_heads + g.n_kv_heads;
    const int head_groups = n_heads / 8;                       // 4 for 28 + 4 heads
    const int m_par = 8 / head_groups;                         // XCDs that share a group of heads: 2
    const int head = (xcd % head_groups) * 8 + (nth & 7);
    const int tile_m = (nth >> 3) * m_par + xcd / head_groups;
    const int m_blk = tile_m * 128;
    if (m_blk >= g.M) return;                                  // the whole workgroup, before any barrier
    const bool is_q = head < g.n_q_heads;
    const int kv_head = head - g.n_q_heads;
    const size_t row_bytes = (size_t)g.K * 2;
    const char* x = reinterpret_cast<const char*>(g.x) + (size_t)m_blk * row_bytes;
    const char* w_head = reinterpret_cast<const char*>(is_q ? g.wq + (size_t)head * 128 * g.K
                                                            : g.wk + (size_t)kv_head * 128 * g.K);
    const char* w_strip = reinterpret_cast<const char*>(g.wv + (size_t)head * kQkvStrip * g.K);
    const h16* bias = is_q ? g.bq : g.bk;
    if (bias) bias += (is_q ? head : kv_head) * 128;
    const int kv_row = g.n_kv_heads * 128;
    const int first = g.d_pos ? *g.d_pos : g.pos;

    auto epilogue = [&](const f32x4 (&acc)[4][4], const f32x4 (&accv)[2], int m0, int wn, int lane) {
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int m = m_blk + m0 + 16 * ((b + 2 * wn) & 3) + (lane & 15);
            if (m >= g.M) continue;
            const float2* trow = g.table + (size_t)m * 64;
            size_t cache_at = 0;
            if (g.k_cache) {
                const int t = first + m;
                cache_at = (size_t)(g.page_table ? g.page_table[t >> 6] * 64 + (t & 63) : t) * kv_row;
            }
#pragma unroll
            for (int a = 0; a < 2; ++a) {
                const int col = 32 * wn + 16 * a + 4 * (lane >> 4);        // the pair is (col, col + 64) of the head
                h16x4 lo, hi;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    lo[r] = to_half(acc[a][b][r]);
                    hi[r] = to_half(acc[a + 2][b][r]);
                }
                if (bias) {
                    const h16x4 blo = *reinterpret_cast<const h16x4*>(bias + col);
                    const h16x4 bhi = *reinterpret_cast<const h16x4*>(bias + col + 64);
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        lo[r] = to_half((float)lo[r] + (float)blo[r]);
                        hi[r] = to_half((float)hi[r] + (float)bhi[r]);
                    }
                }
                const float4 cs01 = *reinterpret_cast<const float4*>(trow + col);
                const float4 cs23 = *reinterpret_cast<const float4*>(trow + col + 2);
                const float cv[4] = {cs01.x, cs01.z, cs23.x, cs23.z};
                const float sv[4] = {cs01.y, cs01.w, cs23.y, cs23.w};
                h16x4 olo, ohi;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const Pair p = rotate((float)lo[r], (float)hi[r], cv[r], sv[r]);
                    olo[r] = to_half(p.lo);
                    ohi[r] = to_half(p.hi);
                }
                if (is_q) {
                    h16* dst = g.q + ((size_t)m * g.n_q_heads + head) * 128 + col;
                    *reinterpret_cast<h16x4*>(dst) = olo;
                    *reinterpret_cast<h16x4*>(dst + 64) = ohi;
                } else {
                    if (g.k) {
                        h16* dst = g.k + (size_t)m * kv_row + kv_head * 128 + col;
                        *reinterpret_cast<h16x4*>(dst) = olo;
                        *reinterpret_cast<h16x4*>(dst + 64) = ohi;
                    }
                    if (g.k_cache) {
                        h16* dst = g.k_cache + cache_at + kv_head * 128 + col;
                        *reinterpret_cast<h16x4*>(dst) = olo;
                        *reinterpret_cast<h16x4*>(dst + 64) = ohi;
                    }
                }
            }
            if (b < 2) {                                                   // the strip of v: product, then bias
                const int col = head * kQkvStrip + 4 * (lane >> 4);
                h16x4 o;
#pragma unroll
                for (int r = 0; r < 4; ++r) o[r] = to_half(accv[b][r]);
                if (g.bv) {
                    const h16x4 bb = *reinterpret_cast<const h16x4*>(g.bv + col);
#pragma unroll
                    for (int r = 0; r < 4; ++r) o[r] = to_half((float)o[r] + (float)bb[r]);
                }
                if (g.v) *reinterpret_cast<h16x4*>(g.v + (size_t)m * kv_row + col) = o;
                if (g.v_cache) *reinterpret_cast<h16x4*>(g.v_cache + cache_at + col) = o;
            }
        }
    };
    mfma_dma64_qkv<F16Op, kStages>(x, w_head, w_strip, g.M - m_blk, (int)row_bytes, epilogue);
}

// The front half of a gated MLP in one GEMM: out = silu(fp16(A Wg^T)) * fp16(A Wu^T). A tile multiplies 256 rows of A
// with 128 rows of Wg and the same 128 rows of Wu (mfma_dma64's two-operand layout), so acc[a] and acc[a + 2] of a
// wave are one output element's gate and up products. Both are rounded to FP16 where the two GEMMs' stores round,
// then the SwiGLU kernel's own function runs on them: the result equals vv_gemm_fp16_dev twice and vv_swiglu_dev
// bit for bit, without gate and up ever going to memory (2 x 547 MB written and read again at 14449 x 18944).
template <int TM>
__device__ __forceinline__ void store_tile16_swiglu(const f32x4 (&acc)[4][TM], h16* __restrict__ out, int M, int N,
                                                    int m0, int n0, int lane) {
    typedef h16 h16x4 __attribute__((ext_vector_type(4)));
    const bool vec = (N % 4 == 0) && ((reinterpret_cast<uintptr_t>(out) & 7u) == 0);
#pragma unroll
    for (int b = 0; b < TM; ++b) {
        const int m = m0 + b * 16 + (lane & 15);
        if (m >= M) continue;
        h16* orow = out + (size_t)m * N;
#pragma unroll
        for (int a = 0; a < 2; ++a) {
            const int n = n0 + a * 16 + 4 * (lane >> 4);
            if (n >= N) continue;
            h16x4 o;
#pragma unroll
            for (int r = 0; r < 4; ++r)
                o[r] = to_half(swiglu1((float)to_half(acc[a][b][r]), (float)to_half(acc[a + 2][b][r])));
            if (vec && n + 3 < N) {
                *reinterpret_cast<h16x4*>(orow + n) = o;
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (n + r < N) orow[n + r] = o[r];
            }
        }
    }
}

__global__ __launch_bounds__(Dma64Shape<256>::kWaves * kWave, 2) void gemm_dma64_swiglu(
    const h16* __restrict__ A, const h16* __restrict__ Wg, const h16* __restrict__ Wu, h16* __restrict__ out, int M,
    int N, int K) {
    constexpr int TM = Dma64Shape<256>::TM;
    auto epilogue = [=](const f32x4 (&acc)[4][TM], int m0, int n0, int lane) {
        store_tile16_swiglu<TM>(acc, out, M, N, m0, n0, lane);
    };
    mfma_dma64<F16Op, 256, 2, 2>(A, Wg, M, N, K * 2, epilogue, Wu);
}

// M == 1: bound by the weight bytes. kSplit waves share an output column (a
// weight row), each streaming a contiguous 1/kSplit of it with non-temporal
// 16-byte loads, four in flight; their sums meet in LDS. Narrow outputs take
// more waves per row so that the chip always has thousands of waves in flight
// (N = 3584, K = 18944: 26.4 us with one wave per row).
template <int kSplit>
__global__ __launch_bounds__(kBlock) void gemv_row(const h16* __restrict__ A,
                                                   const h16* __restrict__ B,
                                                   h16* __restrict__ C, int N, int K, float alpha,
                                                   float beta) {
    constexpr int kRows = kWavesPerBlock / kSplit;      // output columns per workgroup
    __shared__ float part[kWavesPerBlock];
    const int wave = wave_in_block(), lane = lane_id();
    const int n = (int)blockIdx.x * kRows + wave / kSplit;
    const int piece = wave % kSplit;
    const int kchunks = K / 8;
    const int per = (kchunks + kSplit - 1) / kSplit;
    const int begin = piece * per, end = min(kchunks, begin + per);
    float acc = 0.0f;
    if (n < N) {
        const Chunk* w = reinterpret_cast<const Chunk*>(B + (size_t)n * K);
        const Chunk* x = reinterpret_cast<const Chunk*>(A);
#pragma unroll 4
        for (int c = begin + lane; c < end; c += kWave) {
            const f32x8 wf = unpack(load_chunk_stream(w + c));
            const f32x8 xf = unpack(load_chunk(x + c));
#pragma unroll
            for (int i = 0; i < 8; ++i) acc = fmaf(xf[i], wf[i], acc);
        }
    }
    acc = wave_sum(acc);
    if constexpr (kSplit > 1) {
        if (lane == 0) part[wave] = acc;
        __syncthreads();
        acc = 0.0f;
#pragma unroll
        for (int p = 0; p < kSplit; ++p) acc += part[(wave / kSplit) * kSplit + p];
    }
    if (n < N && piece == 0 && lane == 0) {
        const h16 old = beta != 0.0f ? C[n] : (h16)0.0f;
        C[n] = to_half(finish(acc, alpha, beta, old));
    }
}

// The same sums for kR consecutive output columns per wave: the activation chunk is loaded once for kR weight
// rows and a wave has kR independent streams in flight, which pays when the rows are long and few (the down
// projection: 3584 columns of K = 18944, 23.9 -> 22.8 us). A column's products are added in gemv_row<kSplit>'s
// order (per lane chunk by chunk, wave_sum, then the pieces in order): the same bits.
template <int kSplit, int kR>
__global__ __launch_bounds__(kBlock) void gemv_rows(const h16* __restrict__ A, const h16* __restrict__ B,
                                                    h16* __restrict__ C, int N, int K, float alpha, float beta) {
    constexpr int kGroups = kWavesPerBlock / kSplit;    // groups of kR columns per workgroup
    __shared__ float part[kGroups][kR][kSplit];
    const int wave = wave_in_block(), lane = lane_id();
    const int group = wave / kSplit, piece = wave % kSplit;
    const int n0 = ((int)blockIdx.x * kGroups + group) * kR;
    const int kchunks = K / 8;
    const int per = (kchunks + kSplit - 1) / kSplit;
    const int begin = piece * per, end = min(kchunks, begin + per);
    float acc[kR];
#pragma unroll
    for (int r = 0; r < kR; ++r) acc[r] = 0.0f;
    if (n0 < N) {
        const Chunk* w[kR];                              // past the last column: that column again, not stored
#pragma unroll
        for (int r = 0; r < kR; ++r) w[r] = reinterpret_cast<const Chunk*>(B + (size_t)min(n0 + r, N - 1) * K);
        const Chunk* x = reinterpret_cast<const Chunk*>(A);
#pragma unroll 2
        for (int c = begin + lane; c < end; c += kWave) {
            const f32x8 xf = unpack(load_chunk(x + c));
#pragma unroll
            for (int r = 0; r < kR; ++r) {
                const f32x8 wf = unpack(load_chunk_stream(w[r] + c));
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[r] = fmaf(xf[i], wf[i], acc[r]);
            }
        }
    }
#pragma unroll
    for (int r = 0; r < kR; ++r) acc[r] = wave_sum(acc[r]);
    if constexpr (kSplit > 1) {
        if (lane == 0) {
#pragma unroll
            for (int r = 0; r < kR; ++r) part[group][r][piece] = acc[r];
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < kR; ++r) {
            acc[r] = 0.0f;
#pragma unroll
            for (int p = 0; p < kSplit; ++p) acc[r] += part[group][r][p];
        }
    }
    if (piece == 0 && lane == 0) {
#pragma unroll
        for (int r = 0; r < kR; ++r) {
            const int n = n0 + r;
            if (n < N) {
                const h16 old = beta != 0.0f ? C[n] : (h16)0.0f;
                C[n] = to_half(finish(acc[r], alpha, beta, old));
            }
        }
    }
}

// One row of the decode step through two or three projections in one launch.
// kFuse == 0: y_i = x W_i^T (+ bias_i) for up to three projections (q/k/v);
// workgroups [first[p], first[p+1]) serve projection p. kFuse == 1: the MLP's
// gate and up projections and its activation, y = silu(x Wg^T) * (x Wu^T), a
// wave group taking the same row of both matrices. Either way every product is
// summed exactly as gemv_row<kSplit> sums it and rounded to FP16 before the
// bias or the activation is applied, so the result equals the separate launches
// bit for bit.
struct GemvProjs {
    const h16* w[3];
    const h16* bias[3];
    h16* y[3];
    int n[3];
    int first[3];
};

template <int kSplit, int kFuse>
__global__ __launch_bounds__(kBlock) void gemv_multi(const h16* __restrict__ A, GemvProjs projs,
                                                     int K) {
    constexpr int kRows = kWavesPerBlock / kSplit;
    __shared__ float part[2][kWavesPerBlock];
    const int wave = wave_in_block(), lane = lane_id();
    const int which = kFuse ? 0 : ((int)blockIdx.x >= projs.first[1]) + ((int)blockIdx.x >= projs.first[2]);
    const int N = projs.n[which];
    const int n = ((int)blockIdx.x - projs.first[which]) * kRows + wave / kSplit;
    const int piece = wave % kSplit;
    const int kchunks = K / 8;
    const int per = (kchunks + kSplit - 1) / kSplit;
    const int begin = piece * per, end = min(kchunks, begin + per);
    float acc = 0.0f, acc2 = 0.0f;
    if (n < N) {
        const Chunk* w = reinterpret_cast<const Chunk*>(projs.w[which] + (size_t)n * K);
        const Chunk* w2 = reinterpret_cast<const Chunk*>(projs.w[1] + (size_t)n * K);
        const Chunk* x = reinterpret_cast<const Chunk*>(A);
#pragma unroll 4
        for (int c = begin + lane; c < end; c += kWave) {
            const f32x8 wf = unpack(load_chunk_stream(w + c));
            const f32x8 xf = unpack(load_chunk(x + c));
#pragma unroll
            for (int i = 0; i < 8; ++i) acc = fmaf(xf[i], wf[i], acc);
            if constexpr (kFuse) {
                const f32x8 uf = unpack(load_chunk_stream(w2 + c));
#pragma unroll
                for (int i = 0; i < 8; ++i) acc2 = fmaf(xf[i], uf[i], acc2);
            }
        }
    }
    acc = wave_sum(acc);
    if constexpr (kFuse) acc2 = wave_sum(acc2);
    if constexpr (kSplit > 1) {
        if (lane == 0) { part[0][wave] = acc; part[1][wave] = acc2; }
        __syncthreads();
        acc = acc2 = 0.0f;
#pragma unroll
        for (int p = 0; p < kSplit; ++p) {
            acc += part[0][(wave / kSplit) * kSplit + p];
            acc2 += part[1][(wave / kSplit) * kSplit + p];
        }
    }
    if (n < N && piece == 0 && lane == 0) {
        h16 o = to_half(acc);
        if constexpr (kFuse) {
            o = to_half(swiglu1((float)o, (float)to_half(acc2)));
        } else if (projs.bias[which]) {
            o = to_half((float)o + (float)projs.bias[which][n]);
        }
        projs.y[which][n] = o;
    }
}

// The waves per weight row vv_gemm_fp16_dev gives a one-row product of width N.
inline int gemv_split(int N) { return N >= 16384 ? 1 : N >= 8192 ? 2 : 4; }

// M <= 64 (a streaming chunk, a few decode rows): bound by the weight bytes, so
// the weights are read exactly once, straight from global memory into MFMA
// operands, and K is split over the eight waves of a workgroup.
//
// A workgroup owns 16 output columns (weight rows) and all M rows. One
// v_mfma_f32_16x16x32_f16 takes 16 weight rows x 32 K values as its A operand
// (lane: row lane % 16, K chunk lane / 16) and 16 activation rows as its B
// operand; kMT such products (M / 16 row tiles) reuse each weight fragment. A
// wave takes every eighth 64-K "line" (two steps: the whole 128-byte cache line
// of each weight row), two lines in flight per iteration; the eight partial
// tiles meet in LDS. The activations (M x K, at most 2.4 MB) come from L1/L2.
// The K order differs from gemm_tile's, so the bits may too (same bounds).
constexpr int kSkinnyWaves = 8;

// Up to three projections of the same activations in one launch (q/k/v,
// gate/up): workgroups [first[p], first[p+1]) serve projection p. A bias, when
// given, is added to the rounded FP16 product and rounded again, exactly as a
// bias-add launch after the GEMM would.
struct SkinnyProjs {
    const void* w[3];
    const void* scales[3];      // INT8: FP32 per weight row; NF4: FP16 absmax per 64 elements; FP16: unused
    const void* mins[3];        // INT4 {scale, min}: FP16 per group, beside the scales
    int gshift;                 // INT4 {scale, min}: log2 of the group size
    const h16* bias[3];
    h16* y[3];
    int n[3];
    int first[3];
    int vec[3];
};

// The eight waves' partial tiles, already in `part`, summed in wave order and stored: register r of lane l of tile
// (w, t) is column n0 + 16 w + 4(l / 16) + r of row 16t + l % 16. A bias, when given, is added to the rounded FP16
// product and rounded again.
template <int kMT, int kWT = 1>
__device__ __forceinline__ void skinny_store(const f32x4 (*part)[kWT * kMT][kWave], h16* __restrict__ C,
                                             const h16* __restrict__ bias, int M, int N, int n0, int vec_store,
                                             float alpha, float beta) {
    const int tid = (int)threadIdx.x, lane = tid & 63, r16 = lane & 15, ks = lane >> 4;
    for (int item = tid >> 6; item < kWT * kMT; item += kSkinnyWaves) {
        const int t = item % kMT;
        f32x4 sum = part[0][item][lane];
#pragma unroll
        for (int w = 1; w < kSkinnyWaves; ++w) {
            const f32x4 p = part[w][item][lane];
#pragma unroll
            for (int r = 0; r < 4; ++r) sum[r] += p[r];
        }
        const int m = 16 * t + r16, n = n0 + 16 * (item / kMT) + 4 * ks;
        if (m < M && n < N) {
            h16* crow = C + (size_t)m * N;
            if (vec_store && n + 3 < N) {
                typedef h16 h16x4 __attribute__((ext_vector_type(4)));
                h16x4 old = {0, 0, 0, 0};
                if (beta != 0.0f) old = *reinterpret_cast<const h16x4*>(crow + n);
                h16x4 o;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    o[r] = to_half(finish(sum[r], alpha, beta, old[r]));
                    if (bias) o[r] = to_half((float)o[r] + (float)bias[n + r]);
                }
                *reinterpret_cast<h16x4*>(crow + n) = o;
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (n + r < N) {
                        const h16 old = beta != 0.0f ? crow[n + r] : (h16)0.0f;
                        h16 o = to_half(finish(sum[r], alpha, beta, old));
                        if (bias) o = to_half((float)o + (float)bias[n + r]);
                        crow[n + r] = o;
                    }
            }
        }
    }
}

template <int kMT, int kFmt>
__global__ __launch_bounds__(kSkinnyWaves * kWave) void gemm_skinny(
    const h16* __restrict__ A, SkinnyProjs projs, int M, int K, float alpha, float beta) {
    __shared__ f32x4 part[kSkinnyWaves][kMT][kWave];
    __shared__ float book[16];
    if constexpr (kFmt == kWoNf4) {
        if (threadIdx.x < 16) book[threadIdx.x] = kNf4Book[threadIdx.x];
        __syncthreads();
    }

    const int tid = (int)threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int r16 = lane & 15, ks = lane >> 4;
    const int which = ((int)blockIdx.x >= projs.first[1]) + ((int)blockIdx.x >= projs.first[2]);
    const WoSource B = {projs.w[which], projs.scales[which], projs.mins[which], projs.gshift};
    const h16* __restrict__ bias = projs.bias[which];
    h16* __restrict__ C = projs.y[which];
    const int N = projs.n[which], vec_store = projs.vec[which];
    const int n0 = ((int)blockIdx.x - projs.first[which]) * 16;
    const int kchunks = K / 8;
    const int nlines = (kchunks + 7) / 8;                 // 64 K values = 8 chunks per line
    const u32x4 zero = {0u, 0u, 0u, 0u};

    const size_t wrow = (size_t)min(n0 + r16, N - 1);
    const u32x4* arow[kMT];
#pragma unroll
    for (int t = 0; t < kMT; ++t)
        arow[t] = reinterpret_cast<const u32x4*>(A + (size_t)min(16 * t + r16, M - 1) * K);

    f32x4 acc[kMT];
#pragma unroll
    for (int t = 0; t < kMT; ++t) acc[t] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    for (int line = wave; line < nlines; line += 2 * kSkinnyWaves) {
        u32x4 w[4], x[kMT][4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {                     // (line, step) = (u / 2, u % 2)
            const int c = (line + (u >> 1) * kSkinnyWaves) * 8 + (u & 1) * 4 + ks;
            const bool live = c < kchunks;
            w[u] = live ? wo_slot<kFmt>(B, book, wrow, K, c) : zero;      // FP16: the 16 bytes as stored
#pragma unroll
            for (int t = 0; t < kMT; ++t) x[t][u] = live ? arow[t][c] : zero;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int t = 0; t < kMT; ++t)
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h16x8, w[u]),
                                                                __builtin_bit_cast(h16x8, x[t][u]),
                                                                acc[t], 0, 0, 0);
    }
#pragma unroll
    for (int t = 0; t < kMT; ++t) part[wave][t][lane] = acc[t];
    __syncthreads();
    skinny_store<kMT>(part, C, bias, M, N, n0, vec_store, alpha, beta);
}

// The same kernel for FP16 weights and whole 64-K lines (K % 64 == 0), with both operands fetched as WHOLE CACHE
// LINES. The fragment a lane needs is 16 bytes of one of sixteen rows: a wave's load touches sixteen half lines, and
// 224 workgroups reading the same activations that way get 8 TB/s out of L2 where whole lines give 19-27 (measured
// with the two patterns alone: 64 rows x 18944, 65.7 us against 20.2); the weights' gather costs the same way. So a
// wave copies its line of the activations and of the weights straight into LDS, eight rows of 128 bytes per
// instruction (lane: row lane / 8, chunk lane % 8 ^ row, so that the fragment reads below find the eight rows of a
// chunk in eight different groups of banks), kDepth lines ahead, and reads the fragments from there. Its LDS is
// its own: no barrier, only its own counters (every copy of the loop is issued by hand, in a fixed number per line,
// so that "all but the last kDepth - 1 lines' copies" is a constant). Same products in the same order: the same
// bits as gemm_skinny. 64 x 3584 x 18944: 97.9 -> 55.7 us; 24 rows: 53.7 -> 36.7; 8 rows: 32.2 -> 27.7.
// kWT: the weights' tiles of sixteen rows a workgroup takes (16 kWT output columns). Two where the projection is
// so wide that one would mean a thousand short-lived workgroups: the activations are then copied once for both.
template <int kMT, int kWT> struct SkinnyLines {
    static constexpr int kTiles = kMT + kWT;                                          // tiles of a line's slot
    static constexpr int kDepth = 10 / kTiles < 4 ? 10 / kTiles : 4;                  // lines in flight per wave
    static constexpr int kLineBytes = kTiles * 2048;                                  // 16 rows x 128 bytes a tile
    static constexpr int kPerLine = 2 * kTiles;                                       // copies per line
    static constexpr size_t kLdsBytes = (size_t)kSkinnyWaves * kDepth * kLineBytes;   // 128 .. 160 KB
    static_assert(kDepth >= 2 && kLdsBytes <= 160 * 1024 &&
                  kLdsBytes >= sizeof(f32x4) * kSkinnyWaves * kWT * kMT * kWave, "the ring fits, and the partial tiles fit into it");
    static_assert((kDepth - 1) * kPerLine < 64, "a wave's six-bit load counter");
};

template <int kMT, int kWT>
__global__ __launch_bounds__(kSkinnyWaves * kWave) void gemm_skinny_lines(
    const h16* __restrict__ A, SkinnyProjs projs, int M, int K, float alpha, float beta) {
    typedef SkinnyLines<kMT, kWT> Shape;
    extern __shared__ __align__(16) char skinny_lds[];
    const int tid = (int)threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r16 = lane & 15, ks = lane >> 4;
    const int which = ((int)blockIdx.x >= projs.first[1]) + ((int)blockIdx.x >= projs.first[2]);
    const h16* __restrict__ W = static_cast<const h16*>(projs.w[which]);
    const h16* __restrict__ bias = projs.bias[which];
    h16* __restrict__ C = projs.y[which];
    const int N = projs.n[which], vec_store = projs.vec[which];
    const int n0 = ((int)blockIdx.x - projs.first[which]) * (16 * kWT);
    const int nlines = K / 64;
    const int mine = (nlines - wave + kSkinnyWaves - 1) / kSkinnyWaves;      // lines wave, wave + 8, ...

    const uint32_t ring = (uint32_t)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) void*)skinny_lds) +
                          (uint32_t)wave * (Shape::kDepth * Shape::kLineBytes);
    // copy j of a line: rows 8 j .. 8 j + 7 of the activations (of the weights' 16 kWT, for the last tiles); this
    // lane: row 8 j + lane / 8, the chunk whose slot in the row is lane % 8
    const char* row[2 * Shape::kTiles];
#pragma unroll
    for (int j = 0; j < 2 * Shape::kTiles; ++j) {
        const int r = 8 * j + (lane >> 3);
        const h16* at = j < 2 * kMT ? A + (size_t)min(r, M - 1) * K : W + (size_t)min(n0 + r - 16 * kMT, N - 1) * K;
        row[j] = reinterpret_cast<const char*>(at) + (((lane & 7) ^ (lane >> 3)) * 16);
    }
    // fragment (tile t, step u): row 16 t + r16 = copy 2 t + r16 / 8, row r16 % 8 of it; chunk 4 u + ks
    uint32_t frag[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) frag[u] = (uint32_t)((r16 >> 3) * 1024 + (r16 & 7) * 128 + (((4 * u + ks) ^ (r16 & 7)) * 16));
    // the copies of this wave's i-th line, into slot i % kDepth
    auto request = [&](int i, int slot) {
        const size_t line = (size_t)(wave + kSkinnyWaves * i) * 128;
        const uint32_t at = ring + (uint32_t)slot * Shape::kLineBytes;
#pragma unroll
        for (int j = 0; j < 2 * Shape::kTiles; ++j)
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                         : : "s"(at + (uint32_t)j * 1024u), "v"(row[j] + line) : "memory", "m0");
    };

    f32x4 acc[kWT][kMT];
#pragma unroll
    for (int w = 0; w < kWT; ++w)
#pragma unroll
        for (int t = 0; t < kMT; ++t) acc[w][t] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int d = 0; d < Shape::kDepth; ++d)
        if (d < mine) request(d, d);
    // (unrolled by the depth, so that a line's LDS slot is fixed)
    for (int i0 = 0; i0 < mine; i0 += Shape::kDepth) {
#pragma unroll
        for (int d = 0; d < Shape::kDepth; ++d) {
            const int i = i0 + d;
            if (i >= mine) break;
            // Line i has landed when only the copies of the kDepth - 1 lines behind it are still counted; towards
            // the end fewer are behind it, and the wave waits for them all (it has nothing left to ask for)
            if (i + Shape::kDepth - 1 < mine)
                asm volatile("s_waitcnt vmcnt(%0)" : : "n"((Shape::kDepth - 1) * Shape::kPerLine) : "memory");
            else
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            const char* slot = skinny_lds + (size_t)wave * (Shape::kDepth * Shape::kLineBytes) + d * Shape::kLineBytes;
            u32x4 x[kMT][2], wf[kWT][2];
#pragma unroll
            for (int w = 0; w < kWT; ++w)
#pragma unroll
                for (int u = 0; u < 2; ++u) wf[w][u] = *reinterpret_cast<const u32x4*>(slot + (kMT + w) * 2048 + frag[u]);
#pragma unroll
            for (int t = 0; t < kMT; ++t)
#pragma unroll
                for (int u = 0; u < 2; ++u) x[t][u] = *reinterpret_cast<const u32x4*>(slot + t * 2048 + frag[u]);
#pragma unroll
            for (int w = 0; w < kWT; ++w)
#pragma unroll
                for (int u = 0; u < 2; ++u)
#pragma unroll
                    for (int t = 0; t < kMT; ++t)
                        acc[w][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h16x8, wf[w][u]),
                                                                           __builtin_bit_cast(h16x8, x[t][u]),
                                                                           acc[w][t], 0, 0, 0);
            if (i + Shape::kDepth < mine) {
                // the slot is read (its fragments are in registers) before it is refilled
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                request(i + Shape::kDepth, d);
            }
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();                                          // every wave is done with its ring: it becomes `part`
    f32x4 (*part)[kWT * kMT][kWave] = reinterpret_cast<f32x4 (*)[kWT * kMT][kWave]>(skinny_lds);
#pragma unroll
    for (int w = 0; w < kWT; ++w)
#pragma unroll
        for (int t = 0; t < kMT; ++t) part[wave][w * kMT + t][lane] = acc[w][t];
    __syncthreads();
    skinny_store<kMT, kWT>(part, C, bias, M, N, n0, vec_store, alpha, beta);
}

template <typename Kernel>
bool allow_big_lds(Kernel kernel, int& ready_device, size_t bytes);

// 17 .. 64 rows against a very wide N (the gate and up projections of a streaming chunk): a
// 128x128 tile spends its time on the 128 rows it copies and multiplies whatever the chunk has, and the K-split
// kernel above has eight waves share 56 lines of a 3584-wide row - seven round trips to memory each, two lines
// deep. Here a workgroup takes 128 output columns and ALL of K: wave w streams the sixteen weight rows of its own
// columns through a ring of its own, kDepth - 1 lines ahead, and the chunk's rows - 16 kMT of them, one ring for
// the workgroup, each wave copying its share of a line - are read by all eight. One barrier per line tells a wave
// that the others' shares of line i have landed and that all have finished with line i - 1, whose slots the next
// copies then take. Every copy is whole cache lines (eight rows of 128 bytes, the chunk XOR the row); every output
// has one accumulator that adds the K steps in order, as the copy-fed tiles do: the same bits as gemm_dma64.
// kW: waves, i.e. 16-column strips, per workgroup (eight: with four, twice the workgroups, it is 12 % slower). Bare
// 16-byte loads of the same bytes in the same grid take 24.9 us for 18944 x 3584 (5.45 TB/s), this kernel 28.5 - 34.5
// from 17 to 64 rows.
template <int kMT, int kW, int kMats = 1> struct StripShape {
    static constexpr int kDepth = kMats == 2 ? 4 : kMT <= 4 ? 6 : 4;                  // ring slots (lines)
    static constexpr int kXCopies = 2 * kMT;                                          // copies of a line of the rows
    static constexpr int kXLine = kMT * 2048, kWLine = 2048 * kMats;      // a wave's sixteen rows of each matrix
    static constexpr size_t kLdsBytes = (size_t)kDepth * (kXLine + kW * kWLine);     // 120 / 144 KB; two matrices: 144 / 160
    static_assert(kLdsBytes <= 160 * 1024, "the rings fit");
    static_assert(kXCopies <= kW || kXCopies % kW == 0, "a wave's share of a line is fixed");
    // copies a wave issues per line: its two of the weights, its share of the rows
    static __device__ __forceinline__ constexpr int x_share(int wave) {
        return kXCopies >= kW ? kXCopies / kW : (wave < kXCopies ? 1 : 0);
    }
    static_assert((kDepth - 2) * (2 * kMats + (kXCopies + kW - 1) / kW) < 64, "a wave's six-bit load counter");
};

// kMats = 2: the gate and up projections at once - W2 is the second matrix, a wave's ring holds sixteen rows of each,
// and the store is the SwiGLU of the two products, each rounded to FP16 first (store_tile16_swiglu's arithmetic: the
// same bits as the two products and vv_swiglu_dev, without gate and up going to memory).
template <int kMT, int kW, int kMats>
__global__ __launch_bounds__(kW * kWave) void gemm_strip(
    const h16* __restrict__ A, const h16* __restrict__ W, const h16* __restrict__ W2, h16* __restrict__ C, int M,
    int N, int K, float alpha, float beta, int vec_store) {
    typedef StripShape<kMT, kW, kMats> Shape;
    extern __shared__ __align__(16) char strip_lds[];
    const int tid = (int)threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r16 = lane & 15, ks = lane >> 4;
    const int n0 = (int)blockIdx.x * (16 * kW) + wave * 16;
    const int nlines = K / 64;
    const uint32_t lds0 = (uint32_t)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) void*)strip_lds);
    const uint32_t x_ring = lds0, w_ring = lds0 + Shape::kDepth * Shape::kXLine + (uint32_t)wave * (Shape::kDepth * Shape::kWLine);
    const char* x_lds = strip_lds;
    const char* w_lds = strip_lds + Shape::kDepth * Shape::kXLine + (size_t)wave * (Shape::kDepth * Shape::kWLine);

    // this lane's part of a copy: row lane / 8 of its eight, the chunk whose slot in the row is lane % 8
    const int r8 = lane >> 3;
    const uint32_t in_row = (uint32_t)(((lane & 7) ^ r8) * 16);
    const char* wrow[2 * kMats];                               // copies 0, 1: W's sixteen rows; 2, 3: W2's
#pragma unroll
    for (int j = 0; j < 2 * kMats; ++j)
        wrow[j] = reinterpret_cast<const char*>((j < 2 ? W : W2) + (size_t)min(n0 + 8 * (j & 1) + r8, N - 1) * K) + in_row;
    constexpr int kMine = Shape::kXCopies >= kW ? Shape::kXCopies / kW : 1;
    const char* xrow[kMine];
    int xcopy[kMine];
#pragma unroll
    for (int q = 0; q < kMine; ++q) {
        xcopy[q] = wave + kW * q;                    // which copy of the line (eight rows each)
        xrow[q] = reinterpret_cast<const char*>(A + (size_t)min(8 * xcopy[q] + r8, M - 1) * K) + in_row;
    }
    const bool copies_x = Shape::kXCopies >= kW || wave < Shape::kXCopies;
    uint32_t frag[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) frag[u] = (uint32_t)((r16 >> 3) * 1024 + (r16 & 7) * 128 + (((4 * u + ks) ^ (r16 & 7)) * 16));

    auto request = [&](int line, int slot) {
        const size_t at = (size_t)line * 128;
#pragma unroll
        for (int j = 0; j < 2 * kMats; ++j)
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                         : : "s"(w_ring + (uint32_t)slot * Shape::kWLine + (uint32_t)j * 1024u), "v"(wrow[j] + at) : "memory", "m0");
        if (copies_x) {
#pragma unroll
            for (int q = 0; q < kMine; ++q)
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                             : : "s"(x_ring + (uint32_t)slot * Shape::kXLine + (uint32_t)xcopy[q] * 1024u), "v"(xrow[q] + at) : "memory", "m0");
        }
    };

    f32x4 acc[kMats][kMT];
#pragma unroll
    for (int g = 0; g < kMats; ++g)
#pragma unroll
        for (int t = 0; t < kMT; ++t) acc[g][t] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int d = 0; d < Shape::kDepth - 1; ++d)
        if (d < nlines) request(d, d);
    // (unrolled by the depth, so that a line's slots are fixed; every wave walks every line: the barriers match)
    for (int i0 = 0; i0 < nlines; i0 += Shape::kDepth) {
#pragma unroll
        for (int d = 0; d < Shape::kDepth; ++d) {
            const int i = i0 + d;
            if (i >= nlines) break;
            // this wave's copies of line i have landed when only those of the kDepth - 2 lines behind it are
            // still counted; towards the end fewer are behind it, and the wave waits for them all
            if (i + Shape::kDepth - 2 < nlines) {
                if (copies_x)
                    asm volatile("s_waitcnt vmcnt(%0)" : : "n"((Shape::kDepth - 2) * (2 * kMats + kMine)) : "memory");
                else
                    asm volatile("s_waitcnt vmcnt(%0)" : : "n"((Shape::kDepth - 2) * 2 * kMats) : "memory");
            } else {
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            }
            __syncthreads();                                  // the others' shares of line i; all are done with line i - 1
            if (i + Shape::kDepth - 1 < nlines) request(i + Shape::kDepth - 1, (d + Shape::kDepth - 1) % Shape::kDepth);
            u32x4 x[kMT][2], wf[kMats][2];
#pragma unroll
            for (int g = 0; g < kMats; ++g)
#pragma unroll
                for (int u = 0; u < 2; ++u)
                    wf[g][u] = *reinterpret_cast<const u32x4*>(w_lds + d * Shape::kWLine + g * 2048 + frag[u]);
#pragma unroll
            for (int t = 0; t < kMT; ++t)
#pragma unroll
                for (int u = 0; u < 2; ++u) x[t][u] = *reinterpret_cast<const u32x4*>(x_lds + d * Shape::kXLine + t * 2048 + frag[u]);
#pragma unroll
            for (int g = 0; g < kMats; ++g)
#pragma unroll
                for (int u = 0; u < 2; ++u)
#pragma unroll
                    for (int t = 0; t < kMT; ++t)
                        acc[g][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h16x8, wf[g][u]),
                                                                           __builtin_bit_cast(h16x8, x[t][u]),
                                                                           acc[g][t], 0, 0, 0);
        }
    }
    // register r of lane l of tile t: column n0 + 4 (l / 16) + r of row 16 t + l % 16
    const int n = n0 + 4 * ks;
    if (n >= N) return;
#pragma unroll
    for (int t = 0; t < kMT; ++t) {
        const int m = 16 * t + r16;
        if (m >= M) continue;
        h16* crow = C + (size_t)m * N;
        typedef h16 h16x4 __attribute__((ext_vector_type(4)));
        if constexpr (kMats == 2) {
            h16x4 o;
#pragma unroll
            for (int r = 0; r < 4; ++r)
                o[r] = to_half(swiglu1((float)to_half(acc[0][t][r]), (float)to_half(acc[1][t][r])));
            if (vec_store && n + 3 < N) {
                *reinterpret_cast<h16x4*>(crow + n) = o;
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (n + r < N) crow[n + r] = o[r];
            }
        } else if (vec_store && n + 3 < N) {
            h16x4 old = {0, 0, 0, 0};
            if (beta != 0.0f) old = *reinterpret_cast<const h16x4*>(crow + n);
            h16x4 o;
#pragma unroll
            for (int r = 0; r < 4; ++r) o[r] = to_half(finish(acc[0][t][r], alpha, beta, old[r]));
            *reinterpret_cast<h16x4*>(crow + n) = o;
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (n + r < N) {
                    const h16 old = beta != 0.0f ? crow[n + r] : (h16)0.0f;
                    crow[n + r] = to_half(finish(acc[0][t][r], alpha, beta, old));
                }
        }
    }
}

// B2 given: C = swiglu(fp16(A B^T), fp16(A B2^T)) (alpha and beta unused)
template <int kMT, int kW, int kMats = 1>
bool launch_strip(const void* A, const void* B, void* C, int M, int N, int K, float alpha, float beta, hipStream_t st,
                  const void* B2 = nullptr) {
    static thread_local int ready = -1;
    typedef StripShape<kMT, kW, kMats> Shape;
    if (!allow_big_lds(gemm_strip<kMT, kW, kMats>, ready, Shape::kLdsBytes)) return false;
    const int vec = (N % 4 == 0) && ((reinterpret_cast<uintptr_t>(C) & 7u) == 0);
    gemm_strip<kMT, kW, kMats><<<dim3((unsigned)((N + 16 * kW - 1) / (16 * kW))), kW * kWave, Shape::kLdsBytes, st>>>(
        static_cast<const h16*>(A), static_cast<const h16*>(B), static_cast<const h16*>(B2), static_cast<h16*>(C), M, N,
        K, alpha, beta, vec);
    return true;
}



// The 64-column tile count below which the weight-streaming kernel beats the
// tile kernel for 17..64 rows (M = 29, N = 18944 is 31 us tiled against 46 us
// streamed; N = 3584, K = 18944 is 136 us against 48 us).
inline bool few_tiles(int N) { return (long)((N + 63) / 64) < 200; }
inline bool skinny_serves(int M, int N) { return M >= 2 && (M <= 16 || (M <= 64 && few_tiles(N))); }

// The shapes gemm() hands to gemm_strip: 17 .. 64 rows of whole 64-K lines against an N too wide for the
// weight-streaming kernel (and not so wide that the 256x256 tiles would fill the chip twice).
inline bool strip_serves(int M, int N, int K) {
    return M > 16 && M <= 64 && K > 0 && K % 64 == 0 && !skinny_serves(M, N) &&
           (long)((M + 255) / 256) * ((N + 255) / 256) < 512;
}

template <int kMT, int kWT>
bool launch_skinny_lines(const h16* A, const SkinnyProjs& projs, int blocks, int M, int K, float alpha, float beta,
                         hipStream_t st) {
    static thread_local int ready = -1;
    if (!allow_big_lds(gemm_skinny_lines<kMT, kWT>, ready, SkinnyLines<kMT, kWT>::kLdsBytes)) return false;
    gemm_skinny_lines<kMT, kWT><<<dim3((unsigned)blocks), kSkinnyWaves * kWave, SkinnyLines<kMT, kWT>::kLdsBytes, st>>>(
        A, projs, M, K, alpha, beta);
    return true;
}

// One projection of up to 16 rows so wide that its 16-column blocks are more than two rounds of workgroups: 32
// columns each (16 x 18944 x 3584: 32.9 -> 30.6 us; with more rows it gains nothing).
inline bool skinny_pairs(const SkinnyProjs& projs, int blocks, int M) {
    return M <= 16 && blocks > 512 && projs.first[1] == blocks && projs.first[2] == blocks;
}

template <int kFmt>
void launch_skinny_as(const h16* A, const SkinnyProjs& projs, int blocks, int M, int K, float alpha,
                      float beta, hipStream_t st) {
    constexpr int kThreads = kSkinnyWaves * kWave;
    const dim3 grid((unsigned)blocks);
    // FP16 weights in whole lines: both operands by whole cache lines through LDS. Should the launch be refused, the
    // plain kernel below serves.
    if (kFmt == kWoF16 && K % 64 == 0) {
        bool aligned = aligned16(A);
        for (int p = 0; p < 3; ++p) aligned = aligned && (projs.w[p] == nullptr || aligned16(projs.w[p]));
        if (aligned && skinny_pairs(projs, blocks, M)) {
            SkinnyProjs wide = projs;
            const int pairs = (blocks + 1) / 2;
            wide.first[1] = wide.first[2] = pairs;
            if (launch_skinny_lines<1, 2>(A, wide, pairs, M, K, alpha, beta, st)) return;
        }
        if (aligned && (M <= 16 ? launch_skinny_lines<1, 1>(A, projs, blocks, M, K, alpha, beta, st)
                        : M <= 32 ? launch_skinny_lines<2, 1>(A, projs, blocks, M, K, alpha, beta, st)
                        : M <= 48 ? launch_skinny_lines<3, 1>(A, projs, blocks, M, K, alpha, beta, st)
                                  : launch_skinny_lines<4, 1>(A, projs, blocks, M, K, alpha, beta, st)))
            return;
    }
    if (M <= 16) gemm_skinny<1, kFmt><<<grid, kThreads, 0, st>>>(A, projs, M, K, alpha, beta);
    else if (M <= 32) gemm_skinny<2, kFmt><<<grid, kThreads, 0, st>>>(A, projs, M, K, alpha, beta);
    else if (M <= 48) gemm_skinny<3, kFmt><<<grid, kThreads, 0, st>>>(A, projs, M, K, alpha, beta);
    else gemm_skinny<4, kFmt><<<grid, kThreads, 0, st>>>(A, projs, M, K, alpha, beta);
}

void launch_skinny(const h16* A, const SkinnyProjs& projs, int blocks, int M, int K, float alpha,
                   float beta, hipStream_t st, int format = kWoF16) {
    if (format == kWoInt8) launch_skinny_as<kWoInt8>(A, projs, blocks, M, K, alpha, beta, st);
    else if (format == kWoNf4) launch_skinny_as<kWoNf4>(A, projs, blocks, M, K, alpha, beta, st);
    else if (format == kWoAwq) launch_skinny_as<kWoAwq>(A, projs, blocks, M, K, alpha, beta, st);
    else launch_skinny_as<kWoF16>(A, projs, blocks, M, K, alpha, beta, st);
}

__global__ __launch_bounds__(kBlock) void gemm_naive(const h16* A, const h16* B, h16* C, int M,
                                                     int N, int K, float alpha, float beta) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= (size_t)M * N) return;
    const int m = (int)(i / N), n = (int)(i % N);
    const h16* a = A + (size_t)m * K;
    const h16* b = B + (size_t)n * K;
    float acc = 0.0f;
    for (int k = 0; k < K; ++k) acc = fmaf((float)a[k], (float)b[k], acc);
    const h16 old = beta != 0.0f ? C[i] : (h16)0.0f;
    C[i] = to_half(finish(acc, alpha, beta, old));
}

template <int BM, int BN, int WM, int WN, int kSlab, int kAhead = 1>
void launch_tile(const void* A, const void* B, void* C, int M, int N, int K, float alpha,
                 float beta, hipStream_t st) {
    const int vec = (N % 4 == 0) && ((reinterpret_cast<uintptr_t>(C) & 7u) == 0);
    const dim3 grid((unsigned)((N + BN - 1) / BN), (unsigned)((M + BM - 1) / BM));
    if (K % kSlab == 0)
        gemm_tile<BM, BN, WM, WN, kSlab, true, kAhead><<<grid, WM * WN * kWave, 0, st>>>(
            static_cast<const h16*>(A), static_cast<const h16*>(B), static_cast<h16*>(C), M, N, K,
            alpha, beta, vec);
    else
        gemm_tile<BM, BN, WM, WN, kSlab, false, kAhead><<<grid, WM * WN * kWave, 0, st>>>(
            static_cast<const h16*>(A), static_cast<const h16*>(B), static_cast<h16*>(C), M, N, K,
            alpha, beta, vec);
}

// 128 KB of LDS per workgroup is above the default limit: raised once per thread, device and kernel.
template <typename Kernel>
bool allow_big_lds(Kernel kernel, int& ready_device, size_t bytes) {
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) return false;
    if (ready_device != device) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)bytes) != hipSuccess) {
            (void)hipGetLastError();
            return false;
        }
        ready_device = device;
    }
    return true;
}

// The part of C that the 256x256 tiles' launch covers when its last round of workgroups would run mostly empty.
// Every XCD takes an eighth of the tiles, 32 at a time, so a launch costs ceil(tiles / 8 / 32) rounds: 57 x 14
// tiles (14449 rows into 3584 columns) are 3.1 rounds and cost four, 8 x 74 (a 2048-row chunk into 18944
// columns) are 2.3 and cost three. The rows - or the columns - that spill into a round of their own go to the
// 128x128 tile instead, whose rounds are short: 0.42 of a 256x256 round when no compute unit gets a second
// workgroup (at most 256 tiles, four stages), 0.6 per 512 tiles otherwise (measured at K = 3584 and 18944).
// 54 rows of tiles in three rounds and the other 625 rows in one short one; 64 columns of tiles in two rounds
// and the other 2560 columns in one short one. {0, 0}: no split pays (at least a twentieth of the time).
struct Dma64Split { int rows, cols; };

Dma64Split dma64_split(int M, int N) {
    const int gx = (N + kDmaTile - 1) / kDmaTile, gy = (M + kDmaTile - 1) / kDmaTile;
    auto rounds = [](long tiles) { return (double)(((tiles + 7) / 8 + 31) / 32); };
    auto rest = [](int m, int n) {
        const long small = (long)((m + 127) / 128) * ((n + 127) / 128);
        return small <= 256 ? 0.42 : 0.6 * (double)((small + 511) / 512);
    };
    double best = rounds((long)gx * gy) * 0.95;
    Dma64Split split = {0, 0};
    for (int r = gy - 1; r >= 1 && r >= gy - 16; --r) {
        const double cost = rounds((long)gx * r) + rest(M - r * kDmaTile, N);
        if (cost < best) {
            best = cost;
            split = {r * kDmaTile, 0};
        }
    }
    for (int c = gx - 1; c >= 1 && c >= gx - 16; --c) {
        const double cost = rounds((long)gy * c) + rest(M, N - c * kDmaTile);
        if (cost < best) {
            best = cost;
            split = {0, c * kDmaTile};
        }
    }
    return split;
}

// C's rows are ldc halves apart: the launch may cover a range of C's columns (B's rows).
template <int kTile, int kStages = 2>
bool launch_dma64(const void* A, const void* B, void* C, int M, int N, int K, int ldc, float alpha, float beta,
                  hipStream_t st) {
    typedef Dma64Shape<kTile, kStages> Shape;
    static thread_local int ready = -1;
    if (!allow_big_lds(gemm_dma64<kTile, kStages>, ready, Shape::kLdsBytes)) return false;
    const int vec = (ldc % 4 == 0) && ((reinterpret_cast<uintptr_t>(C) & 7u) == 0);
    gemm_dma64<kTile, kStages><<<dim3(dma64_grid<kTile>(M, N)), Shape::kWaves * kWave, Shape::kLdsBytes, st>>>(
        static_cast<const h16*>(A), static_cast<const h16*>(B), static_cast<h16*>(C), M, N, K, ldc, alpha, beta, vec);
    return true;
}

// The 128x128 tile: fed by copies straight into LDS when K is a multiple of 64 (four stages deep when no
// compute unit gets a second workgroup to fill its waits, two otherwise), through registers otherwise.
bool dma128_alone(int M, int N) { return (long)((M + 127) / 128) * ((N + 127) / 128) <= 256; }

bool launch_dma128(const void* A, const void* B, void* C, int M, int N, int K, int ldc, float alpha, float beta,
                   hipStream_t st) {
    return dma128_alone(M, N) ? launch_dma64<128, 4>(A, B, C, M, N, K, ldc, alpha, beta, st)
                              : launch_dma64<128, 2>(A, B, C, M, N, K, ldc, alpha, beta, st);
}

// The 64x64 tile fed the same way, for more than 64 rows (up to 64 the small-M kernels and their bit-for-bit
// contract with the register-fed tiles rule): eight stages while every workgroup has a compute unit to itself.
bool dma64_serves(int M, int K) { return M > 64 && K % (kDma64SlabBytes / 2) == 0; }

bool launch_dma_small(const void* A, const void* B, void* C, int M, int N, int K, float alpha, float beta,
                      hipStream_t st) {
    const long tiles = (long)((M + 63) / 64) * ((N + 63) / 64);
    return tiles <= 256 ? launch_dma64<64, 8>(A, B, C, M, N, K, N, alpha, beta, st)
                        : launch_dma64<64, 4>(A, B, C, M, N, K, N, alpha, beta, st);
}

void launch_128(const void* A, const void* B, void* C, int M, int N, int K, float alpha, float beta,
                hipStream_t st) {
    if (K % (kDma64SlabBytes / 2) == 0 && launch_dma128(A, B, C, M, N, K, N, alpha, beta, st)) return;
    launch_tile<128, 128, 2, 2, 64, 2>(A, B, C, M, N, K, alpha, beta, st);
}

bool launch_dma(const void* A, const void* B, void* C, int M, int N, int K, float alpha, float beta,
                hipStream_t st) {
    static thread_local int ready32 = -1;
    const int vec = (N % 4 == 0) && ((reinterpret_cast<uintptr_t>(C) & 7u) == 0);
    if (K % (kDma64SlabBytes / 2) == 0) {
        const h16* a = static_cast<const h16*>(A);
        const h16* b = static_cast<const h16*>(B);
        h16* c = static_cast<h16*>(C);
        const Dma64Split sp = dma64_split(M, N);
        // the 128x128 part first: should its launch be refused, the 256x256 tiles take everything
        if (sp.cols && launch_dma128(a, b + (size_t)sp.cols * K, c + sp.cols, M, N - sp.cols, K, N, alpha, beta, st))
            return launch_dma64<256>(a, b, c, M, sp.cols, K, N, alpha, beta, st) ||
                   launch_dma64<256>(a, b, c, M, N, K, N, alpha, beta, st);
        if (!launch_dma64<256>(a, b, c, sp.rows ? sp.rows : M, N, K, N, alpha, beta, st)) return false;
        if (sp.rows) launch_128(a + (size_t)sp.rows * K, b, c + (size_t)sp.rows * N, M - sp.rows, N, K, alpha, beta, st);
        return true;
    }
    if (!allow_big_lds(gemm_dma, ready32, kDmaLdsBytes)) return false;
    const dim3 grid((unsigned)((N + kDmaTile - 1) / kDmaTile), (unsigned)((M + kDmaTile - 1) / kDmaTile));
    gemm_dma<<<grid, kDmaWaves * kWave, kDmaLdsBytes, st>>>(
        static_cast<const h16*>(A), static_cast<const h16*>(B), static_cast<h16*>(C), M, N, K, alpha,
        beta, vec);
    return true;
}

// k128: the 128x128 tile through registers (the tile of vv_gemm_fp16_tile_dev); k128dma: that tile fed by copies
// straight into LDS where K allows, what the automatic choice takes.
enum TileChoice : int { kAuto = 0, k128 = 1, k64 = 2, k32 = 3, k256 = 4, k256regs = 5, k128dma = 6 };

vv_status_t gemm(const void* A, const void* B, void* C, int M, int N, int K, float alpha,
                 float beta, void* stream, int choice, bool allow_gemv) {
    if (!A || !B || !C) return VV_ERR_NULL_PTR;
    if (M <= 0 || N <= 0) return VV_OK;
    if (K < 0) return VV_ERR_INVALID_ARG;
    hipStream_t st = as_stream(stream);
    const h16* a = static_cast<const h16*>(A);
    const h16* b = static_cast<const h16*>(B);
    h16* c = static_cast<h16*>(C);

    // K == 0 goes here too (C = beta * C): the tile kernels' first slab fetch is
    // unconditional and would read past an empty operand.
    if (K == 0 || K % 8 != 0 || !aligned16(A) || !aligned16(B)) {
        const size_t blocks = ((size_t)M * N + kBlock - 1) / kBlock;
        gemm_naive<<<dim3((unsigned)blocks), kBlock, 0, st>>>(a, b, c, M, N, K, alpha, beta);
        return launch_status();
    }
    if (allow_gemv && M == 1) {
        const int split = gemv_split(N);
        if (split == 4 && K >= 8192) {                  // few long rows: two per wave
            gemv_rows<4, 2><<<dim3((unsigned)((N + 1) / 2)), kBlock, 0, st>>>(a, b, c, N, K, alpha, beta);
            return launch_status();
        }
        const dim3 grid((unsigned)((N + kWavesPerBlock / split - 1) / (kWavesPerBlock / split)));
        if (split == 1) gemv_row<1><<<grid, kBlock, 0, st>>>(a, b, c, N, K, alpha, beta);
        else if (split == 2) gemv_row<2><<<grid, kBlock, 0, st>>>(a, b, c, N, K, alpha, beta);
        else gemv_row<4><<<grid, kBlock, 0, st>>>(a, b, c, N, K, alpha, beta);
        return launch_status();
    }
    // Up to 64 rows: the weight-streaming kernel, unless there are more than 16
    // rows and enough 64-wide column tiles to fill the chip.
    if (allow_gemv && skinny_serves(M, N)) {
        SkinnyProjs projs = {};
        projs.w[0] = b;
        projs.y[0] = c;
        projs.n[0] = N;
        projs.vec[0] = (N % 4 == 0) && ((reinterpret_cast<uintptr_t>(C) & 7u) == 0);
        const int blocks = (N + 15) / 16;
        projs.first[1] = projs.first[2] = blocks;
        launch_skinny(a, projs, blocks, M, K, alpha, beta, st);
        return launch_status();
    }
    const bool auto_choice = choice == kAuto;
    if (choice == kAuto) {
        // The largest tile that still fills the 256 compute units: 256x256
        // (eight waves, the fewest L1 and LDS bytes per MFMA; fed by direct
        // global-to-LDS copies when K is a multiple of 32, through registers
        // otherwise) from two full rounds of workgroups on, 128x128 from one
        // round on.
        const long wg256 = (long)((M + 255) / 256) * ((N + 255) / 256);
        const long wg128 = (long)((M + 127) / 128) * ((N + 127) / 128);
        // (copy-fed, four stages deep, the 128x128 tile already pays with half the compute units busy:
        // 1024 x 3584 x 3584 in 31 us as 224 tiles of 128, 50 us as 896 tiles of 64; at 112 tiles the 64s win)
        const long enough128 = K % (kDma64SlabBytes / 2) == 0 ? 128 : 256;
        // (17 .. 64 rows arrive here when N is too wide for the weight-streaming kernel; should the kernel below be
        // refused: one row of 128x128 tiles)
        const bool rows128 = M > 64 || (M > 16 && K % (kDma64SlabBytes / 2) == 0);
        // 17 .. 64 rows that arrive here (N too wide for the weight-streaming kernel), whole 64-K lines: the kernel
        // that gives a workgroup 128 columns and all of K (24 x 18944 x 3584: 29 us; 33 us as one row of 128x128 tiles,
        // which still serve 65 .. 128 rows, where it gains nothing; 46 us as 64-wide tiles)
        if (strip_serves(M, N, K) && (M <= 32 ? launch_strip<2, 8>(A, B, C, M, N, K, alpha, beta, st)
                                               : launch_strip<4, 8>(A, B, C, M, N, K, alpha, beta, st)))
            return launch_status();
        choice = wg256 >= 512 ? k256 : (rows128 && wg128 >= enough128) ? k128dma : (M > 32) ? k64 : k32;
    }
    switch (choice) {
        case k128dma: launch_128(A, B, C, M, N, K, alpha, beta, st); break;
        case k256:
            if (K % (kDmaSlabBytes / 2) == 0 && launch_dma(A, B, C, M, N, K, alpha, beta, st)) break;
            [[fallthrough]];
        case k256regs: launch_tile<256, 256, 2, 4, 32, 2>(A, B, C, M, N, K, alpha, beta, st); break;
        case k128: launch_tile<128, 128, 2, 2, 64, 2>(A, B, C, M, N, K, alpha, beta, st); break;
        case k64:
            if (auto_choice && dma64_serves(M, K) && launch_dma_small(A, B, C, M, N, K, alpha, beta, st)) break;
            launch_tile<64, 64, 2, 2, 64, 1>(A, B, C, M, N, K, alpha, beta, st);
            break;
        default:   launch_tile<32, 64, 1, 2, 64, 1>(A, B, C, M, N, K, alpha, beta, st); break;
    }
    return launch_status();
}

// C = rope(fp16(A W^T) + bias) in the GEMM's store, for the shapes the LDS-tiled kernels serve: the
// same tile rule as gemm() above 64 rows, except that the two small tiles give way to 64 x 128 (the
// narrowest block that holds a whole head; all tile shapes add K in the same order). false: nothing
// launched (up to 64 rows, where gemm() streams the weights in another K order, and odd K).
template <int BM, int BN, int WM, int WN, int kSlab, int kAhead>
void launch_tile_rope(const h16* A, const h16* B, const h16* bias, const float2* table, h16* C, int M, int N,
                      int K, hipStream_t st) {
    const dim3 grid((unsigned)((N + BN - 1) / BN), (unsigned)((M + BM - 1) / BM));
    if (K % kSlab == 0)
        gemm_tile_rope<BM, BN, WM, WN, kSlab, true, kAhead><<<grid, WM * WN * kWave, 0, st>>>(
            A, B, bias, table, C, M, N, K, 1.0f, 0.0f);
    else
        gemm_tile_rope<BM, BN, WM, WN, kSlab, false, kAhead><<<grid, WM * WN * kWave, 0, st>>>(
            A, B, bias, table, C, M, N, K, 1.0f, 0.0f);
}

template <int kTile, int kStages = 2>
bool launch_dma64_rope(const h16* A, const h16* B, const h16* bias, const float2* table, h16* C, int M, int N,
                       int K, int ldc, hipStream_t st) {
    typedef Dma64Shape<kTile, kStages> Shape;
    static thread_local int ready = -1;
    if (!allow_big_lds(gemm_dma64_rope<kTile, kStages>, ready, Shape::kLdsBytes)) return false;
    gemm_dma64_rope<kTile, kStages><<<dim3(dma64_grid<kTile>(M, N)), Shape::kWaves * kWave, Shape::kLdsBytes, st>>>(
        A, B, bias, table, C, M, N, K, ldc, 1.0f, 0.0f);
    return true;
}

bool launch_dma128_rope(const h16* A, const h16* B, const h16* bias, const float2* table, h16* C, int M, int N,
                        int K, int ldc, hipStream_t st) {
    return dma128_alone(M, N) ? launch_dma64_rope<128, 4>(A, B, bias, table, C, M, N, K, ldc, st)
                              : launch_dma64_rope<128, 2>(A, B, bias, table, C, M, N, K, ldc, st);
}

void launch_128_rope(const h16* A, const h16* B, const h16* bias, const float2* table, h16* C, int M, int N, int K,
                     hipStream_t st) {
    if (K % (kDma64SlabBytes / 2) == 0 && launch_dma128_rope(A, B, bias, table, C, M, N, K, N, st)) return;
    launch_tile_rope<128, 128, 2, 2, 64, 2>(A, B, bias, table, C, M, N, K, st);
}

bool gemm_rope(const h16* A, const h16* B, const h16* bias, const float2* table, h16* C, int M, int N, int K,
               hipStream_t st, int choice) {
    if (M <= 64 || K <= 0 || K % 8 != 0) return false;
    if (choice == kAuto) {
        const long wg256 = (long)((M + 255) / 256) * ((N + 255) / 256);
        const long wg128 = (long)((M + 127) / 128) * ((N + 127) / 128);
        const long enough128 = K % (kDma64SlabBytes / 2) == 0 ? 128 : 256;       // as in gemm()
        choice = wg256 >= 512 ? k256 : wg128 >= enough128 ? k128dma : k64;
        // gemm() gives these shapes to the copy-fed 64x64 tile, which is narrower than a head: the caller runs
        // the two steps one after the other (on the 16x16x32 instruction like that tile, so the bits agree)
        if (choice == k64 && dma64_serves(M, K)) return false;
    }
    if (choice == k256 && K % (kDmaSlabBytes / 2) == 0) {
        static thread_local int ready32 = -1;
        if (K % (kDma64SlabBytes / 2) == 0) {
            const Dma64Split sp = dma64_split(M, N);         // the split of gemm(), so the same bits
            if (sp.cols && launch_dma128_rope(A, B + (size_t)sp.cols * K, bias ? bias + sp.cols : nullptr, table,
                                              C + sp.cols, M, N - sp.cols, K, N, st)) {
                if (launch_dma64_rope<256>(A, B, bias, table, C, M, sp.cols, K, N, st) ||
                    launch_dma64_rope<256>(A, B, bias, table, C, M, N, K, N, st))
                    return true;
            } else if (launch_dma64_rope<256>(A, B, bias, table, C, sp.rows ? sp.rows : M, N, K, N, st)) {
                if (sp.rows)
                    launch_128_rope(A + (size_t)sp.rows * K, B, bias, table + (size_t)sp.rows * 64,
                                    C + (size_t)sp.rows * N, M - sp.rows, N, K, st);
                return true;
            }
        } else if (allow_big_lds(gemm_dma_rope, ready32, kDmaLdsBytes)) {
            const dim3 grid((unsigned)((N + kDmaTile - 1) / kDmaTile), (unsigned)((M + kDmaTile - 1) / kDmaTile));
            gemm_dma_rope<<<grid, kDmaWaves * kWave, kDmaLdsBytes, st>>>(A, B, bias, table, C, M, N, K, 1.0f, 0.0f);
            return true;
        }
    }
    if (choice == k256 || choice == k256regs) launch_tile_rope<256, 256, 2, 4, 32, 2>(A, B, bias, table, C, M, N, K, st);
    else if (choice == k128dma) launch_128_rope(A, B, bias, table, C, M, N, K, st);
    else if (choice == k128) launch_tile_rope<128, 128, 2, 2, 64, 2>(A, B, bias, table, C, M, N, K, st);
    else launch_tile_rope<64, 128, 2, 2, 64, 1>(A, B, bias, table, C, M, N, K, st);
    return true;
}

// The fused q / k / v tile serves: 7 query heads per KV head of 128 channels in groups of eight heads, more than 64
// rows of whole 64-half slabs (where the separate calls run their copy-fed 16x16x32 tiles too: same K order).
bool qkv_serves(int M, int n_q_heads, int n_kv_heads, int head_dim, int K) {
    const int n_heads = n_q_heads + n_kv_heads;
    return head_dim == 128 && n_kv_heads * 128 == n_heads * kQkvStrip && n_heads % 8 == 0 && 8 % (n_heads / 8) == 0 &&
           dma64_serves(M, K) && (size_t)K * 2 * 144 < 0x7fffffffu;
}

template <int kStages>
bool launch_qkv(const QkvArgs& g, hipStream_t st) {
    typedef QkvShape<kStages> Shape;
    static thread_local int ready = -1;
    if (!allow_big_lds(gemm_dma64_qkv<kStages>, ready, Shape::kLdsBytes)) return false;
    const int n_heads = g.n_q_heads + g.n_kv_heads;
    const int m_par = 8 / (n_heads / 8);
    const int gy = (g.M + 127) / 128;
    const unsigned grid = 64u * (unsigned)((gy + m_par - 1) / m_par);
    gemm_dma64_qkv<kStages><<<dim3(grid), Shape::kWaves * kWave, Shape::kLdsBytes, st>>>(g);
    return true;
}

int forced_tile() {
    static const int v = [] {
        const char* e = getenv("VV_GEMM_TILE");
        return e ? atoi(e) : 0;
    }();
    return (v >= 0 && v <= 6) ? v : 0;
}

}  // namespace
}  // namespace vv

// For linear_wonly.hip: y[M][N] = A[M][K] x W^T for one INT4 {scale, min} weight through the small-M kernel (the
// format is not one of the public entry point's), or VV_ERR_UNSUPPORTED (nothing launched) where
// vv_gemm_fp16_dev would not hand the shape to that kernel.
__attribute__((visibility("hidden")))
vv_status_t vv_skinny_int4_minmax(const void* A, const void* w, const void* scales, const void* mins, int gshift,
                                  void* y, int M, int N, int K, void* stream) {
    if (M < 9 || M > 64 || K % 8 != 0 || !vv::aligned16(A) || !vv::skinny_serves(M, N) ||
        (reinterpret_cast<uintptr_t>(w) & 3u) || (reinterpret_cast<uintptr_t>(scales) & 1u) ||
        (reinterpret_cast<uintptr_t>(mins) & 1u))
        return VV_ERR_UNSUPPORTED;
    vv::SkinnyProjs p = {};
    p.w[0] = w;
    p.scales[0] = scales;
    p.mins[0] = mins;
    p.gshift = gshift;
    p.y[0] = static_cast<vv::h16*>(y);
    p.n[0] = N;
    p.vec[0] = (N % 4 == 0) && ((reinterpret_cast<uintptr_t>(y) & 7u) == 0);
    const int blocks = (N + 15) / 16;
    p.first[1] = p.first[2] = blocks;
    vv::launch_skinny(static_cast<const vv::h16*>(A), p, blocks, M, K, 1.0f, 0.0f, vv::as_stream(stream), vv::kWoAwq);
    return vv::launch_status();
}

// For linear_wonly.hip: y[M][N] = A[M][K] x W^T, 9 <= M <= 64, for one weight in a weight-only format through the
// LDS-tiled kernel with the weight dequantised on its way in: no scratch, the bits of dequantise + vv_gemm_fp16_dev
// where that tiles. VV_ERR_UNSUPPORTED (nothing launched) outside what it covers.
template <int kFmt>
static vv_status_t tile_wo(const vv::h16* A, const vv::WoSource& B, vv::h16* C, int M, int N, int K, hipStream_t st) {
    const int vec = (N % 4 == 0) && ((reinterpret_cast<uintptr_t>(C) & 7u) == 0);
    // Unpacking a slot costs about what multiplying it does: four waves per tile even when two would hold the rows
    // (measured faster for every format from 17 rows on; the tile shape changes no bit).
    const dim3 grid((unsigned)((N + 63) / 64), (unsigned)((M + 63) / 64));
    if (K % 64 == 0) vv::gemm_tile_wo<64, 64, 2, 2, 64, true, kFmt><<<grid, 4 * vv::kWave, 0, st>>>(A, B, C, M, N, K, vec);
    else vv::gemm_tile_wo<64, 64, 2, 2, 64, false, kFmt><<<grid, 4 * vv::kWave, 0, st>>>(A, B, C, M, N, K, vec);
    return vv::launch_status();
}

__attribute__((visibility("hidden")))
vv_status_t vv_gemm_tile_weight_only(int format, const void* A, const void* w, const void* scales, const void* mins,
                                     int gshift, void* y, int M, int N, int K, void* stream) {
    if (M < 9 || M > 64 || N <= 0 || K <= 0 || K % 8 != 0 || !vv::aligned16(A) || vv::skinny_serves(M, N))
        return VV_ERR_UNSUPPORTED;
    const uintptr_t at = reinterpret_cast<uintptr_t>(w);
    if ((format == vv::kWoInt8 ? (at & 7u) : (at & 3u)) != 0) return VV_ERR_UNSUPPORTED;
    const vv::WoSource B = {w, scales, mins, gshift};
    const vv::h16* a = static_cast<const vv::h16*>(A);
    vv::h16* c = static_cast<vv::h16*>(y);
    hipStream_t st = vv::as_stream(stream);
    if (format == vv::kWoInt8) return tile_wo<vv::kWoInt8>(a, B, c, M, N, K, st);
    if (format == vv::kWoNf4) return tile_wo<vv::kWoNf4>(a, B, c, M, N, K, st);
    if (format == vv::kWoAwq) return tile_wo<vv::kWoAwq>(a, B, c, M, N, K, st);
    return VV_ERR_UNSUPPORTED;
}

// rope.hip: x[rows][heads][128] = rope(x + bias), cos/sin from a vv_rope_table_dev table.
vv_status_t vv_rope128_from_table(void* x, const void* bias, const void* table, int rows, int heads, void* stream);
// rope.hip: two tensors of heads_a and heads_b heads rotated in one launch.
vv_status_t vv_rope128_pair_from_table(void* a, void* b, const void* table, int rows, int heads_a, int heads_b,
                                       void* stream);

extern "C" {

vv_status_t vv_gemm_fp16_dev(const void* A, const void* B, void* C, int M, int N, int K,
                             float alpha, float beta, void* stream) {
    return vv::gemm(A, B, C, M, N, K, alpha, beta, stream, vv::forced_tile(), true);
}

/* Declines (nothing launched) whatever vv_gemm_fp16_dev would not hand to the
 * weight-streaming kernel, so that the caller's fallback (vv_gemm_fp16_dev, then
 * vv_bias_add_dev, per projection) and this entry point always give the same bits. */
vv_status_t vv_skinny_linear_dev(const void* A, int format, const vv_skinny_proj_t* projs, int n_proj,
                                 int M, int K, float alpha, void* stream) {
    if (!A || !projs) return VV_ERR_NULL_PTR;
    if ((format != vv::kWoF16 && format != vv::kWoInt8 && format != vv::kWoNf4) || n_proj < 1 || n_proj > 3 ||
        M < 9 || M > 64 || K <= 0 || K % 8 != 0 || !vv::aligned16(A))
        return VV_ERR_UNSUPPORTED;
    vv::SkinnyProjs p = {};
    int blocks = 0;
    for (int i = 0; i < 3; ++i) {
        p.first[i] = blocks;
        if (i >= n_proj) continue;
        if (!projs[i].w || !projs[i].y || (format != vv::kWoF16 && !projs[i].scales)) return VV_ERR_NULL_PTR;
        // the widest load per weight row: 16 bytes of FP16, 8 of int8, 4 of NF4 codes
        const uintptr_t at = reinterpret_cast<uintptr_t>(projs[i].w);
        const bool placed = format == vv::kWoF16 ? (at & 15u) == 0 : format == vv::kWoInt8 ? (at & 7u) == 0 : (at & 3u) == 0;
        if (projs[i].N <= 0 || !vv::skinny_serves(M, projs[i].N) || !placed ||
            (format != vv::kWoF16 && (reinterpret_cast<uintptr_t>(projs[i].scales) & (format == vv::kWoInt8 ? 3u : 1u))))
            return VV_ERR_UNSUPPORTED;
        p.w[i] = projs[i].w;
        p.scales[i] = projs[i].scales;
        p.bias[i] = static_cast<const vv::h16*>(projs[i].bias);
        p.y[i] = static_cast<vv::h16*>(projs[i].y);
        p.n[i] = projs[i].N;
        p.vec[i] = (projs[i].N % 4 == 0) && ((reinterpret_cast<uintptr_t>(projs[i].y) & 7u) == 0);
        blocks += (projs[i].N + 15) / 16;
    }
    vv::launch_skinny(static_cast<const vv::h16*>(A), p, blocks, M, K, alpha, 0.0f, vv::as_stream(stream), format);
    return vv::launch_status();
}

vv_status_t vv_gemv_multi_dev(const void* x, const vv_skinny_proj_t* projs, int n_proj, int K,
                              void* stream) {
    if (!x || !projs) return VV_ERR_NULL_PTR;
    if (n_proj < 1 || n_proj > 3 || K <= 0 || K % 8 != 0 || !vv::aligned16(x)) return VV_ERR_UNSUPPORTED;
    vv::GemvProjs p = {};
    const int split = vv::gemv_split(projs[0].N);
    const int rows = vv::kWavesPerBlock / split;
    int blocks = 0;
    for (int i = 0; i < 3; ++i) {
        p.first[i] = blocks;
        if (i >= n_proj) continue;
        if (!projs[i].w || !projs[i].y) return VV_ERR_NULL_PTR;
        if (projs[i].N <= 0 || vv::gemv_split(projs[i].N) != split || !vv::aligned16(projs[i].w))
            return VV_ERR_UNSUPPORTED;
        p.w[i] = static_cast<const vv::h16*>(projs[i].w);
        p.bias[i] = static_cast<const vv::h16*>(projs[i].bias);
        p.y[i] = static_cast<vv::h16*>(projs[i].y);
        p.n[i] = projs[i].N;
        blocks += (projs[i].N + rows - 1) / rows;
    }
    for (int i = n_proj; i < 3; ++i) p.w[i] = p.w[0];
    const vv::h16* a = static_cast<const vv::h16*>(x);
    hipStream_t st = vv::as_stream(stream);
    if (split == 1) vv::gemv_multi<1, 0><<<dim3((unsigned)blocks), vv::kBlock, 0, st>>>(a, p, K);
    else if (split == 2) vv::gemv_multi<2, 0><<<dim3((unsigned)blocks), vv::kBlock, 0, st>>>(a, p, K);
    else vv::gemv_multi<4, 0><<<dim3((unsigned)blocks), vv::kBlock, 0, st>>>(a, p, K);
    return vv::launch_status();
}

vv_status_t vv_gemv_swiglu_dev(const void* x, const void* w_gate, const void* w_up, void* y, int N,
                               int K, void* stream) {
    if (!x || !w_gate || !w_up || !y) return VV_ERR_NULL_PTR;
    if (N <= 0) return VV_OK;
    if (K <= 0 || K % 8 != 0 || !vv::aligned16(x) || !vv::aligned16(w_gate) || !vv::aligned16(w_up))
        return VV_ERR_UNSUPPORTED;
    vv::GemvProjs p = {};
    p.w[0] = static_cast<const vv::h16*>(w_gate);
    p.w[1] = p.w[2] = static_cast<const vv::h16*>(w_up);
    p.y[0] = static_cast<vv::h16*>(y);
    p.n[0] = N;
    const int split = vv::gemv_split(N);
    const int rows = vv::kWavesPerBlock / split;
    const dim3 grid((unsigned)((N + rows - 1) / rows));
    p.first[1] = p.first[2] = (int)grid.x;
    const vv::h16* a = static_cast<const vv::h16*>(x);
    hipStream_t st = vv::as_stream(stream);
    if (split == 1) vv::gemv_multi<1, 1><<<grid, vv::kBlock, 0, st>>>(a, p, K);
    else if (split == 2) vv::gemv_multi<2, 1><<<grid, vv::kBlock, 0, st>>>(a, p, K);
    else vv::gemv_multi<4, 1><<<grid, vv::kBlock, 0, st>>>(a, p, K);
    return vv::launch_status();
}

vv_status_t vv_gemm_bias_rope_dev(const void* A, const void* W, const void* bias, void* C, int M,
                                  int n_heads, int head_dim, int K, const void* rope_table, void* stream) {
    if (!A || !W || !C || !rope_table) return VV_ERR_NULL_PTR;
    if (M <= 0 || n_heads <= 0) return VV_OK;
    if (K < 0) return VV_ERR_INVALID_ARG;
    if (head_dim != 128 || !vv::aligned16(C) || !vv::aligned16(rope_table) || (bias && !vv::aligned16(bias)))
        return VV_ERR_UNSUPPORTED;
    const int N = n_heads * 128;
    if (vv::aligned16(A) && vv::aligned16(W) &&
        vv::gemm_rope(static_cast<const vv::h16*>(A), static_cast<const vv::h16*>(W),
                      static_cast<const vv::h16*>(bias), static_cast<const float2*>(rope_table),
                      static_cast<vv::h16*>(C), M, N, K, vv::as_stream(stream), vv::forced_tile()))
        return vv::launch_status();
    // What the fused kernels do not cover: the two steps one after the other, on the same table.
    const vv_status_t s = vv::gemm(A, W, C, M, N, K, 1.0f, 0.0f, stream, vv::forced_tile(), true);
    if (s != VV_OK) return s;
    return vv_rope128_from_table(C, bias, rope_table, M, n_heads, stream);
}

vv_status_t vv_gemm_qkv_rope_dev(const void* x, const void* wq, const void* wk, const void* wv, const void* bq,
                                 const void* bk, const void* bv, void* q, void* k, void* v, int M, int n_q_heads,
                                 int n_kv_heads, int head_dim, int K, const void* rope_table, void* k_cache,
                                 void* v_cache, const int* page_table, int pos, const int* d_pos, void* stream) {
    if (!x || !wq || !wk || !wv || !q || !rope_table) return VV_ERR_NULL_PTR;
    if ((!k || !v) && (!k_cache || !v_cache)) return VV_ERR_NULL_PTR;
    if ((k_cache == nullptr) != (v_cache == nullptr)) return VV_ERR_NULL_PTR;
    if (M <= 0 || n_q_heads <= 0 || n_kv_heads <= 0) return VV_OK;
    if (K < 0 || pos < 0) return VV_ERR_INVALID_ARG;
    const void* aligned[] = {q, k, v, k_cache, v_cache, rope_table, bq, bk, bv};
    for (const void* p : aligned)
        if (p && !vv::aligned16(p)) return VV_ERR_UNSUPPORTED;
    if (head_dim != 128) return VV_ERR_UNSUPPORTED;
    // From the row count at which the q projection fills the chip with 256x256 tiles (two rounds of them), the
    // separate launches are faster (14449 rows: 490 against 539 us); below, the equal tiles are (2048 rows: 73
    // against 109 us).
    const bool big_tiles = (long)((M + 255) / 256) * ((n_q_heads * 128 + 255) / 256) >= 512 && k && v;
    if (vv::forced_tile() == 0 && !big_tiles && vv::qkv_serves(M, n_q_heads, n_kv_heads, head_dim, K) && vv::aligned16(x) &&
        vv::aligned16(wq) && vv::aligned16(wk) && vv::aligned16(wv)) {
        typedef const vv::h16* H;
        const vv::QkvArgs g = {static_cast<H>(x), static_cast<H>(wq), static_cast<H>(wk), static_cast<H>(wv),
                               static_cast<H>(bq), static_cast<H>(bk), static_cast<H>(bv),
                               static_cast<const float2*>(rope_table), static_cast<vv::h16*>(q),
                               static_cast<vv::h16*>(k), static_cast<vv::h16*>(v), static_cast<vv::h16*>(k_cache),
                               static_cast<vv::h16*>(v_cache), page_table, d_pos, pos, M, K, n_q_heads, n_kv_heads};
        // up to 256 tiles a workgroup has its compute unit to itself and asks for its slabs four ahead
        const long tiles = (long)((M + 127) / 128) * (n_q_heads + n_kv_heads);
        if (tiles <= 256 ? vv::launch_qkv<4>(g, vv::as_stream(stream)) : vv::launch_qkv<2>(g, vv::as_stream(stream)))
            return vv::launch_status();
    }
    // Everything else: the separate launches, through the caller's k and v buffers.
    if (!k || !v) return VV_ERR_UNSUPPORTED;
    // 2 .. 64 rows (a streaming chunk): the three projections with their biases in one launch of the weight-streaming
    // kernel - which is what each of the calls below would run for its own projection, so the same bits - then one
    // rotation of the q and k rows, then the append: three launches instead of seven.
    const int nq_cols = n_q_heads * head_dim, nkv_cols = n_kv_heads * head_dim;
    if (vv::forced_tile() == 0 && M >= 2 && M <= 64 && K > 0 && K % 8 == 0 && vv::skinny_serves(M, nq_cols) &&
        vv::skinny_serves(M, nkv_cols) && vv::aligned16(x) && vv::aligned16(wq) && vv::aligned16(wk) && vv::aligned16(wv)) {
        vv::SkinnyProjs p = {};
        const void* ws[3] = {wq, wk, wv};
        const void* bs[3] = {bq, bk, bv};
        void* ys[3] = {q, k, v};
        int blocks = 0;
        for (int i = 0; i < 3; ++i) {
            p.first[i] = blocks;
            p.w[i] = ws[i];
            p.bias[i] = static_cast<const vv::h16*>(bs[i]);
            p.y[i] = static_cast<vv::h16*>(ys[i]);
            p.n[i] = i == 0 ? nq_cols : nkv_cols;
            p.vec[i] = 1;                                      // whole heads of 128 columns, 16-byte aligned rows
            blocks += (p.n[i] + 15) / 16;
        }
        vv::launch_skinny(static_cast<const vv::h16*>(x), p, blocks, M, K, 1.0f, 0.0f, vv::as_stream(stream));
        vv_status_t s = vv::launch_status();
        if (s != VV_OK) return s;
        s = vv_rope128_pair_from_table(q, k, rope_table, M, n_q_heads, n_kv_heads, stream);
        if (s != VV_OK || !k_cache) return s;
        return vv_kv_store_dev(k, v, k_cache, v_cache, nullptr, nullptr, nullptr, false, n_kv_heads, head_dim, pos,
                               d_pos, M, 0, page_table, stream);
    }
    vv_status_t s = vv_gemm_bias_rope_dev(x, wq, bq, q, M, n_q_heads, head_dim, K, rope_table, stream);
    if (s != VV_OK) return s;
    s = vv_gemm_bias_rope_dev(x, wk, bk, k, M, n_kv_heads, head_dim, K, rope_table, stream);
    if (s != VV_OK) return s;
    const int nkv = n_kv_heads * head_dim;
    s = vv::gemm(x, wv, v, M, nkv, K, 1.0f, 0.0f, stream, vv::forced_tile(), true);
    if (s != VV_OK) return s;
    if (bv && (s = vv_bias_add_dev(v, bv, M, nkv, stream)) != VV_OK) return s;
    if (k_cache)
        return vv_kv_store_dev(k, v, k_cache, v_cache, nullptr, nullptr, nullptr, false, n_kv_heads, head_dim, pos,
                               d_pos, M, 0, page_table, stream);
    return VV_OK;
}

vv_status_t vv_gemm_swiglu_dev(const void* A, const void* w_gate, const void* w_up, void* gate, void* up,
                               void* out, int M, int N, int K, void* stream) {
    if (!A || !w_gate || !w_up || !out) return VV_ERR_NULL_PTR;
    if (M <= 0 || N <= 0) return VV_OK;
    if (K < 0) return VV_ERR_INVALID_ARG;
    // The fused tile where vv_gemm_fp16_dev itself would run its copy-fed 16x16x32 tiles (they all add K in one
    // order, whatever their size): more than 64 rows of whole 64-half slabs at 16-byte aligned addresses.
    if (vv::dma64_serves(M, K) && K > 0 && N <= (1 << 29) && vv::aligned16(A) && vv::aligned16(w_gate) &&
        vv::aligned16(w_up)) {
        typedef vv::Dma64Shape<256, 2> Shape;
        static thread_local int ready = -1;
        if (vv::allow_big_lds(vv::gemm_dma64_swiglu, ready, Shape::kLdsBytes)) {
            vv::gemm_dma64_swiglu<<<dim3(vv::dma64_grid<256>(M, 2 * N)), Shape::kWaves * vv::kWave, Shape::kLdsBytes,
                                    vv::as_stream(stream)>>>(
                static_cast<const vv::h16*>(A), static_cast<const vv::h16*>(w_gate),
                static_cast<const vv::h16*>(w_up), static_cast<vv::h16*>(out), M, N, K);
            return vv::launch_status();
        }
    }
    // One row: the decode step's own fused launch (equal to the three calls by its own contract).
    if (M == 1 && vv_gemv_swiglu_dev(A, w_gate, w_up, out, N, K, stream) == VV_OK) return VV_OK;
    // 17 .. 64 rows against a very wide N (a streaming chunk): where vv_gemm_fp16_dev itself would stream 128 columns a
    // workgroup, the same kernel on both matrices at once, SwiGLU in its store
    if (vv::forced_tile() == 0 && vv::strip_serves(M, N, K) && vv::aligned16(A) && vv::aligned16(w_gate) &&
        vv::aligned16(w_up) &&
        (M <= 32 ? vv::launch_strip<2, 8, 2>(A, w_gate, out, M, N, K, 1.0f, 0.0f, vv::as_stream(stream), w_up)
                 : vv::launch_strip<4, 8, 2>(A, w_gate, out, M, N, K, 1.0f, 0.0f, vv::as_stream(stream), w_up)))
        return vv::launch_status();
    // Everything else: the three steps one after the other, through the caller's gate and up buffers.
    if (!gate || !up || (size_t)M * (size_t)N > 0x7fffffffu) return VV_ERR_UNSUPPORTED;
    vv_status_t s = vv::gemm(A, w_gate, gate, M, N, K, 1.0f, 0.0f, stream, vv::forced_tile(), true);
    if (s != VV_OK) return s;
    s = vv::gemm(A, w_up, up, M, N, K, 1.0f, 0.0f, stream, vv::forced_tile(), true);
    if (s != VV_OK) return s;
    return vv_swiglu_dev(gate, up, out, M * N, stream);
}

vv_status_t vv_gemm_fp16_tile_dev(const void* A, const void* B, void* C, int M, int N, int K,
                                  float alpha, float beta, void* stream) {
    // 9..64 rows: whatever vv_gemm_fp16_dev runs there. The small-M entry point is held to this
    // one bit for bit (device.h:464-468), and the weight-streaming kernel adds K in its own order.
    if (M >= 9 && M <= 64) return vv::gemm(A, B, C, M, N, K, alpha, beta, stream, vv::forced_tile(), true);
    return vv::gemm(A, B, C, M, N, K, alpha, beta, stream, vv::k128, false);
}

}  // extern "C"
