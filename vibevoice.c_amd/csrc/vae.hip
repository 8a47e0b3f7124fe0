// The matrix-core part of the batched, streaming Conv-VAE encoder ops (the direct and im2col
// convolutions, the context copy and the per-column 1/rms are not built here: their entry points
// answer VV_ERR_UNSUPPORTED). FP16 activations, channel-first
// and packed along time; the items of a launch sit side by side in one
// [C][ld] buffer and only the convolutions know where one ends (a descriptor
// passed by value). No output's arithmetic depends on where its item sits, on
// how a stream was cut into chunks, or on which workgroup computes it: every
// sum runs in one fixed order, and an FP16 rounding happens wherever a chain of
// separate kernels would have stored an intermediate. So batching, chunking
// and fusing change no bit.
//
//   vae_mixer_vec  RMSNorm -> depthwise conv -> gamma residual, fused, 16-byte accesses
//   vae_gemm       the FFN (A x B, B K-major) and connector (A x B^T) GEMMs on
//                  v_mfma_f32_16x16x32_f16: 128x128 or 64x64 tile, four waves,
//                  64 K per LDS stage; a K-major B is transposed on its way
//                  into LDS (and RMS-normalised there when asked); epilogues
//                  bias+GELU, bias+gamma-residual, bias, bias+row scatter; whole
//                  tiles leave through LDS as 16-byte stores
#include "vv_common.hpp"

namespace vv {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

typedef vv_vae_conv_desc_t Desc;
typedef vv_vae_conv_item_t Item;

// The fused mixer's tile: 64 columns x 32 channels per workgroup, depthwise kernels of up to 16 taps.
constexpr int kMixT = 64, kMixC = 32, kMixMaxK = 16;

// The mixer (RMSNorm -> depthwise conv -> gamma residual) for packed buffers whose rows and items start on
// 16-byte boundaries (ld % 8 == 0, every in_off % 8 == 0): thread (channel, chunk) moves eight columns with
// one 16-byte access per tensor; a fixed order per sum and an FP16 rounding where separate kernels would
// have stored one.
__global__ __launch_bounds__(kBlock) void vae_mixer_vec(Desc d, const h16* __restrict__ xin, h16* __restrict__ xout,
                                                        int64_t ld, const float* __restrict__ rinv, int64_t T_total,
                                                        const h16* __restrict__ nw, const h16* __restrict__ cw,
                                                        const h16* __restrict__ cb, const h16* __restrict__ gamma, int C,
                                                        int k) {
    const int item = (int)blockIdx.z;
    const Item& it = d.it[item];
    const int t0 = (int)blockIdx.x * kMixT;
    if (t0 >= it.in_len) return;
    const int c0 = (int)blockIdx.y * kMixC;
    const int H = k - 1;
    // nv[channel][kMixMaxK + column]: the tile's columns start 16-byte aligned, the halo sits just below them
    __shared__ __attribute__((aligned(16))) h16 nv[kMixC][kMixMaxK + kMixT];
    const int cl = (int)threadIdx.x >> 3, ch = (int)threadIdx.x & 7;
    const int c = c0 + cl, t = t0 + 8 * ch;
    const bool row_ok = c < C;
    const bool whole = row_ok && t + 8 <= it.in_len;               // the chunk lies inside the item
    const float wn = row_ok ? (float)nw[c] : 0.0f;
    h16x8 xv;
#pragma unroll
    for (int j = 0; j < 8; ++j) xv[j] = (h16)0.0f;
    h16x8 nchunk = xv;
    if (row_ok && t < it.in_len) {
        const int64_t col = it.in_off + t;
        const h16* src = xin + (size_t)c * ld + col;
        if (whole) {
            xv = *reinterpret_cast<const h16x8*>(src);
            const f32x4 r0 = *reinterpret_cast<const f32x4*>(rinv + col), r1 = *reinterpret_cast<const f32x4*>(rinv + col + 4);
#pragma unroll
            for (int j = 0; j < 8; ++j) nchunk[j] = to_half(((float)xv[j] * (j < 4 ? r0[j] : r1[j - 4])) * wn);
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j)
                if (t + j < it.in_len) {
                    xv[j] = src[j];
                    nchunk[j] = to_half(((float)xv[j] * rinv[col + j]) * wn);
                }
        }
    }
    *reinterpret_cast<h16x8*>(&nv[cl][kMixMaxK + 8 * ch]) = nchunk;
    // the halo: H columns to the left of the tile, from the item's input or its carried context
    const h16* tl = static_cast<const h16*>(it.tail_in);
    for (int e = (int)threadIdx.x; e < kMixC * H; e += kBlock) {
        const int hl = e / H, q = e - hl * H;
        const int hc = c0 + hl;
        h16 out = (h16)0.0f;
        if (hc < C) {
            const int p = t0 - H + q;
            if (p >= 0) {
                const int64_t col = it.in_off + p;
                out = to_half(((float)xin[(size_t)hc * ld + col] * rinv[col]) * (float)nw[hc]);
            } else {
                const int tp = it.have + p;
                if (tl && tp >= 0)
                    out = to_half(((float)tl[(size_t)hc * d.cap + tp] * rinv[T_total + (int64_t)item * d.cap + tp]) *
                                  (float)nw[hc]);
            }
        }
        nv[hl][kMixMaxK - H + q] = out;
    }
    __syncthreads();
    if (!row_ok || t >= it.in_len) return;
    float win[8 + kMixMaxK - 1];
#pragma unroll
    for (int j = 0; j < 8 + kMixMaxK - 1; ++j) win[j] = j < 8 + H ? (float)nv[cl][kMixMaxK - H + 8 * ch + j] : 0.0f;
    float sum[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) sum[j] = 0.0f;
#pragma unroll
    for (int kk = 0; kk < kMixMaxK; ++kk) {
        if (kk < k) {
            const float wv = (float)cw[c * k + kk];
#pragma unroll
            for (int j = 0; j < 8; ++j) sum[j] = __builtin_fmaf(wv, win[j + kk], sum[j]);
        }
    }
    const float bias = cb ? (float)cb[c] : 0.0f;
    const float g = gamma ? (float)gamma[c] : 0.0f;
    h16x8 o;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        float sj = sum[j];
        if (cb) sj += bias;
        const float yv = (float)to_half(sj);
        o[j] = gamma ? to_half(__builtin_fmaf(yv, g, (float)xv[j])) : to_half((float)xv[j] + yv);
    }
    h16* dst = xout + (size_t)c * ld + it.in_off + t;
    if (whole) {
        *reinterpret_cast<h16x8*>(dst) = o;
    } else {
#pragma unroll
        for (int j = 0; j < 8; ++j)
            if (t + j < it.in_len) dst[j] = o[j];
    }
}

// ── GEMMs on the matrix cores ───────────────────────────────────────────────

enum { kEpiBiasGelu = 0, kEpiBiasResid = 1, kEpiBias = 2, kEpiRows = 3, kEpiAlphaBeta = 4 };

struct GemmOut {
    h16* c;
    int64_t ldc;
    const h16* bias;       // per row (NN epilogues) or per column (rows epilogue)
    const h16* gamma;
    float alpha, beta;
    vv_vae_rows_t rows;
};

__device__ __forceinline__ float vae_gelu(float x) { return 0.5f * x * (1.0f + erff(x * 0.7071067811865476f)); }

// FP32 -> FP16 by truncation of the mantissa, subnormal results flushed to a
// signed zero, overflow to infinity.
__device__ __forceinline__ h16 trunc_half(float f) {
    const uint32_t u = __builtin_bit_cast(uint32_t, f);
    const uint32_t sign = (u >> 16) & 0x8000u;
    const int e = (int)((u >> 23) & 0xFF) - 127 + 15;
    const uint32_t frac = (u >> 13) & 0x3FFu;
    uint16_t h;
    if (e <= 0) h = (uint16_t)sign;
    else if (e >= 31) h = (uint16_t)(sign | 0x7C00u);
    else h = (uint16_t)(sign | ((uint32_t)e << 10) | frac);
    return __builtin_bit_cast(h16, h);
}

// The value of C[r][.] from its accumulated product and, for the forms that add to C, its old value.
template <int kEpi>
__device__ __forceinline__ h16 gemm_value(const GemmOut& o, float acc, int r, h16 old) {
    if constexpr (kEpi == kEpiAlphaBeta) {
        float v = o.alpha * acc;
        if (o.beta != 0.0f) v = __builtin_fmaf(o.beta, (float)old, v);
        return to_half(v);
    } else if constexpr (kEpi == kEpiBias) {
        return to_half(acc + (o.bias ? (float)o.bias[r] : 0.0f));
    } else {
        float v = (float)to_half(acc);
        if (o.bias) v = (float)to_half(v + (float)o.bias[r]);
        if constexpr (kEpi == kEpiBiasGelu) return to_half(vae_gelu(v));
        const float xv = (float)old;
        return o.gamma ? to_half(__builtin_fmaf(v, (float)o.gamma[r], xv)) : to_half(xv + v);
    }
}

template <int kEpi>
__device__ __forceinline__ void gemm_finish(const GemmOut& o, float acc, int r, int c) {
    if constexpr (kEpi == kEpiRows) {
        h16 y = to_half(acc);
        if (o.bias) y = to_half((float)y + (float)o.bias[c]);
        if (o.rows.mode == VV_VAE_ROWS_PLAIN) {
            o.c[(size_t)r * o.ldc + c] = y;
            return;
        }
        int s = 0;
        while (s + 1 < o.rows.n && r >= o.rows.seg[s + 1].row0) ++s;
        h16* dst = static_cast<h16*>(o.rows.seg[s].dst) + (size_t)(r - o.rows.seg[s].row0) * o.rows.seg[s].ld + c;
        if (o.rows.mode == VV_VAE_ROWS_STORE) *dst = y;
        else if (o.rows.mode == VV_VAE_ROWS_STORE_TRUNC) *dst = trunc_half((float)y);
        else *dst = trunc_half((float)*dst + (float)y);
        return;
    }
    const size_t off = (size_t)r * o.ldc + c;
    const bool reads = kEpi == kEpiBiasResid || (kEpi == kEpiAlphaBeta && o.beta != 0.0f);
    o.c[off] = gemm_value<kEpi>(o, acc, r, reads ? o.c[off] : (h16)0.0f);
}

constexpr int kGK = 64;          // K per LDS stage: two MFMA steps
constexpr int kGLd = kGK + 8;    // LDS row stride in halves: 144 bytes, 16-byte aligned, rows on different banks

// C[M][P] = A[M][K] (row stride lda) x B, B either [P][K] (kNN false, row stride ldb) or [K][P] (kNN true, row
// stride ldb; optionally RMS-normalised while staged). kT x kT outputs per workgroup (64 or 128), four waves of
// kT/2 x kT/2. Every output adds its K products 32 at a time in K order whatever the tile, so the tile changes no bit.
template <bool kNN, int kEpi, int kT>
__global__ __launch_bounds__(kBlock) void vae_gemm(const h16* __restrict__ A, int64_t lda, const h16* __restrict__ B,
                                                   int64_t ldb, int M, int K, int P, const float* __restrict__ rinv,
                                                   const h16* __restrict__ nw, GemmOut out) {
    constexpr int kF = kT / 32;                 // 16x16 MFMA tiles per wave along each side
    constexpr int kCLd = kT + 8;                // row stride of the result tile
    static_assert(2 * kT * kGLd >= kT * kCLd, "the result tile fits over the operand stages");
    __shared__ __attribute__((aligned(16))) h16 lds[2 * kT * kGLd];
    h16 (*As)[kGLd] = reinterpret_cast<h16 (*)[kGLd]>(lds);
    h16 (*Bs)[kGLd] = reinterpret_cast<h16 (*)[kGLd]>(lds + kT * kGLd);
    const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int r16 = lane & 15, kq = lane >> 4;
    const int row_base = (int)blockIdx.y * kT, col_base = (int)blockIdx.x * kT;
    const bool a_vec = (lda & 7) == 0 && (reinterpret_cast<uintptr_t>(A) & 15u) == 0;
    const bool b_vec = (ldb & 7) == 0 && (reinterpret_cast<uintptr_t>(B) & 15u) == 0;

    f32x4 acc[kF][kF];
#pragma unroll
    for (int i = 0; i < kF; ++i)
#pragma unroll
        for (int j = 0; j < kF; ++j) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    // Staging is split in two so that the next stage's global loads are in flight while this stage multiplies:
    // fetch_* bring a stage's chunks into registers, put_* write them to LDS after the products of the stage before.
    constexpr int kRowChunks = kT * 8 / kBlock;          // chunks per thread of a K-contiguous operand's stage
    constexpr int kHalves = kT / 64;
    // K-contiguous rows of `src` (row stride ld): kT rows x 8 chunks of 8.
    auto fetch_rows = [&](const h16* src, int64_t ld, bool vec, int base, int limit, int k0, h16x8 (&reg)[kRowChunks]) {
#pragma unroll
        for (int u = 0; u < kRowChunks; ++u) {
            const int e = tid + u * kBlock;
            const int r = e >> 3, c = (e & 7) * 8;
            const int gr = base + r;
            if (vec && gr < limit && k0 + c + 8 <= K) {
                reg[u] = *reinterpret_cast<const h16x8*>(src + (size_t)gr * ld + k0 + c);
            } else {
#pragma unroll
                for (int t = 0; t < 8; ++t)
                    reg[u][t] = (gr < limit && k0 + c + t < K) ? src[(size_t)gr * ld + k0 + c + t] : (h16)0.0f;
            }
        }
    };
    auto put_rows = [&](const h16x8 (&reg)[kRowChunks], h16 (*dst)[kGLd]) {
#pragma unroll
        for (int u = 0; u < kRowChunks; ++u) {
            const int e = tid + u * kBlock;
            *reinterpret_cast<h16x8*>(&dst[e >> 3][(e & 7) * 8]) = reg[u];
        }
    };
    // K-major B: thread (kg, c) takes K rows 2 kg, 2 kg + 1 of the stage and columns 8 c .. 8 c + 7 (of every 64),
    // and writes the eight (k, k + 1) pairs into Bs[column][k]. The 16-byte K groups of a Bs row are XOR-ed with
    // the column's (column / 8) % 8, which spreads a wave's 64 pair writes over all 64 banks.
    const int kg = tid >> 3;
    float col_rinv[kHalves][8];                          // 1 / rms of this thread's columns: the same for every stage
    if constexpr (kNN) {
#pragma unroll
        for (int half = 0; half < kHalves; ++half)
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const int gc = col_base + half * 64 + (tid & 7) * 8 + t;
                col_rinv[half][t] = (nw && gc < P) ? rinv[gc] : 0.0f;
            }
    }
    auto fetch_kmajor = [&](int k0, h16x8 (&reg)[kHalves][2]) {
#pragma unroll
        for (int half = 0; half < kHalves; ++half) {
            const int gc = col_base + half * 64 + (tid & 7) * 8;
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const int gk = k0 + 2 * kg + u;
                if (b_vec && gk < K && gc + 8 <= P) {
                    reg[half][u] = *reinterpret_cast<const h16x8*>(B + (size_t)gk * ldb + gc);
                } else {
#pragma unroll
                    for (int t = 0; t < 8; ++t)
                        reg[half][u][t] = (gk < K && gc + t < P) ? B[(size_t)gk * ldb + gc + t] : (h16)0.0f;
                }
            }
        }
    };
    auto put_kmajor = [&](int k0, h16x8 (&reg)[kHalves][2]) {
        const int at = (((kg >> 2) ^ (tid & 7)) << 3) + 2 * (kg & 3);       // (column / 8) % 8 == tid & 7 for all of them
#pragma unroll
        for (int half = 0; half < kHalves; ++half) {
            const int c = half * 64 + (tid & 7) * 8;
            if (nw) {
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    const int gk = k0 + 2 * kg + u;
                    const float wn_k = gk < K ? (float)nw[gk] : 0.0f;
#pragma unroll
                    for (int t = 0; t < 8; ++t)        // zero operands (past K or P) stay zero: 0 * x * 0
                        reg[half][u][t] = to_half(((float)reg[half][u][t] * col_rinv[half][t]) * wn_k);
                }
            }
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const h16x2 pair = {reg[half][0][t], reg[half][1][t]};
                *reinterpret_cast<h16x2*>(&Bs[c + t][at]) = pair;
            }
        }
    };

    h16x8 ra[kRowChunks], rb_rows[kNN ? 1 : kRowChunks], rb_k[kNN ? kHalves : 1][2];
    fetch_rows(A, lda, a_vec, row_base, M, 0, ra);
    if constexpr (kNN) fetch_kmajor(0, rb_k);
    else fetch_rows(B, ldb, b_vec, col_base, P, 0, rb_rows);
    for (int k0 = 0; k0 < K; k0 += kGK) {
        put_rows(ra, As);
        if constexpr (kNN) put_kmajor(k0, rb_k);
        else put_rows(rb_rows, Bs);
        __syncthreads();
        if (k0 + kGK < K) {
            fetch_rows(A, lda, a_vec, row_base, M, k0 + kGK, ra);
            if constexpr (kNN) fetch_kmajor(k0 + kGK, rb_k);
            else fetch_rows(B, ldb, b_vec, col_base, P, k0 + kGK, rb_rows);
        }
#pragma unroll
        for (int ks = 0; ks < kGK / 32; ++ks) {
            h16x8 af[kF], bf[kF];
#pragma unroll
            for (int i = 0; i < kF; ++i)
                af[i] = *reinterpret_cast<const h16x8*>(&As[wm * (kT / 2) + i * 16 + r16][ks * 32 + kq * 8]);
#pragma unroll
            for (int j = 0; j < kF; ++j) {
                const int col = wn * (kT / 2) + j * 16 + r16;
                const int group = kNN ? ((ks * 4 + kq) ^ ((col >> 3) & 7)) : ks * 4 + kq;
                bf[j] = *reinterpret_cast<const h16x8*>(&Bs[col][group * 8]);
            }
#pragma unroll
            for (int i = 0; i < kF; ++i)
#pragma unroll
                for (int j = 0; j < kF; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }
    // register r of lane l: row 4 (l / 16) + r of the A tile, column l % 16 of the B tile
    bool through_lds = false;
    if constexpr (kEpi != kEpiRows)
        through_lds = row_base + kT <= M && col_base + kT <= P && (out.ldc & 7) == 0 &&
                      (reinterpret_cast<uintptr_t>(out.c) & 15u) == 0;
    if (through_lds) {
        // A whole tile whose rows are 16-byte aligned: the results meet in LDS (over the operand stages, free after
        // the loop's last barrier) and leave as 16-byte stores; the forms that add to C bring the old tile in the same way.
        h16 (*Ct)[kCLd] = reinterpret_cast<h16 (*)[kCLd]>(lds);
        h16* cbase = out.c + (size_t)row_base * out.ldc + col_base;
        const bool reads = kEpi == kEpiBiasResid || (kEpi == kEpiAlphaBeta && out.beta != 0.0f);
        constexpr int kChunksPerRow = kT / 8;
        if (reads) {
#pragma unroll
            for (int u = 0; u < kT * kChunksPerRow / kBlock; ++u) {
                const int e = tid + u * kBlock;
                const int r = e / kChunksPerRow, c = (e % kChunksPerRow) * 8;
                *reinterpret_cast<h16x8*>(&Ct[r][c]) = *reinterpret_cast<const h16x8*>(cbase + (size_t)r * out.ldc + c);
            }
            __syncthreads();
        }
#pragma unroll
        for (int i = 0; i < kF; ++i)
#pragma unroll
            for (int j = 0; j < kF; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int lr = wm * (kT / 2) + i * 16 + 4 * kq + r, lc = wn * (kT / 2) + j * 16 + r16;
                    if constexpr (kEpi != kEpiRows)
                        Ct[lr][lc] = gemm_value<kEpi>(out, acc[i][j][r], row_base + lr, reads ? Ct[lr][lc] : (h16)0.0f);
                }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < kT * kChunksPerRow / kBlock; ++u) {
            const int e = tid + u * kBlock;
            const int r = e / kChunksPerRow, c = (e % kChunksPerRow) * 8;
            *reinterpret_cast<h16x8*>(cbase + (size_t)r * out.ldc + c) = *reinterpret_cast<const h16x8*>(&Ct[r][c]);
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < kF; ++i)
#pragma unroll
        for (int j = 0; j < kF; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = row_base + wm * (kT / 2) + i * 16 + 4 * kq + r;
                const int col = col_base + wn * (kT / 2) + j * 16 + r16;
                if (row < M && col < P) gemm_finish<kEpi>(out, acc[i][j][r], row, col);
            }
}

// The 128 tile halves the operand bytes a product pulls through L2; the 64 tile keeps small problems on enough
// workgroups. Either gives the same bits.
template <bool kNN, int kEpi>
void launch_vae_gemm(const h16* A, int64_t lda, const h16* B, int64_t ldb, int M, int K, int P, const float* rinv,
                     const h16* nw, const GemmOut& out, hipStream_t st, int tile = 0) {
    const long big = (long)((M + 127) / 128) * ((P + 127) / 128);
    if (tile == 128 || (tile == 0 && M >= 128 && P >= 128 && big >= 512)) {
        const dim3 grid((unsigned)((P + 127) / 128), (unsigned)((M + 127) / 128));
        vae_gemm<kNN, kEpi, 128><<<grid, kBlock, 0, st>>>(A, lda, B, ldb, M, K, P, rinv, nw, out);
    } else {
        const dim3 grid((unsigned)((P + 63) / 64), (unsigned)((M + 63) / 64));
        vae_gemm<kNN, kEpi, 64><<<grid, kBlock, 0, st>>>(A, lda, B, ldb, M, K, P, rinv, nw, out);
    }
}

__global__ __launch_bounds__(kBlock) void vae_f32_to_f16(const float* __restrict__ in, h16* __restrict__ out, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) out[i] = to_half(in[i]);
}

int desc_max(const Desc* d, bool out) {
    int m = 0;
    for (int i = 0; i < d->n; ++i) {
        const int v = out ? d->it[i].out_len : d->it[i].in_len;
        if (v > m) m = v;
    }
    return m;
}

}  // namespace
}  // namespace vv

extern "C" {

vv_status_t vv_vae_conv_dev(const vv_vae_conv_desc_t* d, const void* x, int64_t ld_in, const void* w, const void* b,
                            void* y, int64_t ld_out, int in_ch, int out_ch, int k, int stride, bool transposed,
                            void* stream) {
    (void)d; (void)x; (void)ld_in; (void)w; (void)b; (void)y; (void)ld_out; (void)in_ch; (void)out_ch; (void)k; (void)stride; (void)transposed; (void)stream;
    return VV_ERR_UNSUPPORTED;      // not built in this backend: nothing is launched
}

vv_status_t vv_vae_tail_dev(const vv_vae_conv_desc_t* d, const void* x, int64_t ld_in, int in_ch, void* stream) {
    (void)d; (void)x; (void)ld_in; (void)in_ch; (void)stream;
    return VV_ERR_UNSUPPORTED;      // not built in this backend: nothing is launched
}

vv_status_t vv_vae_rms_dev(const void* x, int64_t ld, int64_t T, int C, float eps, float* rinv,
                           const vv_vae_conv_desc_t* d, void* stream) {
    (void)x; (void)ld; (void)T; (void)C; (void)eps; (void)rinv; (void)d; (void)stream;
    return VV_ERR_UNSUPPORTED;      // not built in this backend: nothing is launched
}

vv_status_t vv_vae_mixer_dev(const vv_vae_conv_desc_t* d, const void* xin, void* xout, int64_t ld, const float* rinv,
                             int64_t T_total, const void* norm_w, const void* conv_w, const void* conv_b,
                             const void* gamma, int C, int k, void* stream) {
    if (!d || !xin || !xout || !rinv || !norm_w || !conv_w) return VV_ERR_NULL_PTR;
    if (k < 1 || k > vv::kMixMaxK || d->n <= 0 || d->n > VV_VAE_MAX_ITEMS || C <= 0) return VV_ERR_INVALID_ARG;
    const int m = vv::desc_max(d, false);
    if (m <= 0) return VV_OK;
    const dim3 grid((unsigned)((m + vv::kMixT - 1) / vv::kMixT), (unsigned)((C + vv::kMixC - 1) / vv::kMixC),
                    (unsigned)d->n);
    typedef const vv::h16* H;
    // 16-byte accesses when every row and every item starts on a 16-byte boundary
    bool vec = (ld & 7) == 0 && vv::aligned16(xin) && vv::aligned16(xout) && vv::aligned16(rinv);
    for (int i = 0; i < d->n && vec; ++i) vec = (d->it[i].in_off & 7) == 0;
    if (!vec) return VV_ERR_UNSUPPORTED;       // only the 16-byte form is built
    vv::vae_mixer_vec<<<grid, vv::kBlock, 0, vv::as_stream(stream)>>>(
        *d, static_cast<H>(xin), static_cast<vv::h16*>(xout), ld, rinv, T_total, static_cast<H>(norm_w),
        static_cast<H>(conv_w), static_cast<H>(conv_b), static_cast<H>(gamma), C, k);
    return vv::launch_status();
}

vv_status_t vv_vae_im2col_dev(const vv_vae_conv_desc_t* d, const void* x, int64_t ld_in, int in_ch, int k, int stride,
                              int64_t p0, int pc, void* col, int64_t ldcol, void* stream) {
    (void)d; (void)x; (void)ld_in; (void)in_ch; (void)k; (void)stride; (void)p0; (void)pc; (void)col; (void)ldcol; (void)stream;
    return VV_ERR_UNSUPPORTED;      // not built in this backend: nothing is launched
}

vv_status_t vv_vae_conv_gemm_dev(const vv_vae_conv_desc_t* d, const void* w, const void* col, int64_t ldcol,
                                 const void* b, void* y, int64_t ld_out, int out_ch, int K, int64_t p0, int pc, int tile,
                                 void* stream) {
    (void)d; (void)w; (void)col; (void)ldcol; (void)b; (void)y; (void)ld_out; (void)out_ch; (void)K; (void)p0; (void)pc; (void)tile; (void)stream;
    return VV_ERR_UNSUPPORTED;      // not built in this backend: nothing is launched
}

vv_status_t vv_vae_gemm_nn_dev(int epilogue, const void* A, const void* B, int64_t ldb, void* C, int64_t ldc, int M,
                               int K, int P, const void* bias, const void* gamma, const float* rinv, const void* norm_w,
                               int tile, void* stream) {
    if (!A || !B || !C) return VV_ERR_NULL_PTR;
    if (M <= 0 || K <= 0 || P <= 0) return VV_ERR_INVALID_ARG;
    if ((norm_w != nullptr) != (rinv != nullptr)) return VV_ERR_INVALID_ARG;
    if (tile != 0 && tile != 64 && tile != 128) return VV_ERR_INVALID_ARG;
    typedef const vv::h16* H;
    vv::GemmOut out = {};
    out.c = static_cast<vv::h16*>(C);
    out.ldc = ldc;
    out.bias = static_cast<H>(bias);
    out.gamma = static_cast<H>(gamma);
    hipStream_t st = vv::as_stream(stream);
    H a = static_cast<H>(A), b = static_cast<H>(B), nw = static_cast<H>(norm_w);
    if (epilogue == VV_VAE_EPI_BIAS_GELU)
        vv::launch_vae_gemm<true, vv::kEpiBiasGelu>(a, K, b, ldb, M, K, P, rinv, nw, out, st, tile);
    else if (epilogue == VV_VAE_EPI_BIAS_RESID)
        vv::launch_vae_gemm<true, vv::kEpiBiasResid>(a, K, b, ldb, M, K, P, rinv, nw, out, st, tile);
    else if (epilogue == VV_VAE_EPI_BIAS)
        vv::launch_vae_gemm<true, vv::kEpiBias>(a, K, b, ldb, M, K, P, rinv, nw, out, st, tile);
    else
        return VV_ERR_INVALID_ARG;
    return vv::launch_status();
}

vv_status_t vv_vae_gemm_tn_dev(const void* A, int64_t lda, const void* B, void* C, int64_t ldc, int M, int N, int K,
                               const void* bias, const vv_vae_rows_t* rows, void* stream) {
    if (!A || !B) return VV_ERR_NULL_PTR;
    if (M <= 0 || N <= 0 || K <= 0) return VV_ERR_INVALID_ARG;
    vv::GemmOut out = {};
    out.rows.mode = VV_VAE_ROWS_PLAIN;
    if (rows) out.rows = *rows;
    if (out.rows.mode == VV_VAE_ROWS_PLAIN && !C) return VV_ERR_NULL_PTR;
    if (out.rows.mode != VV_VAE_ROWS_PLAIN &&
        (out.rows.mode < 0 || out.rows.mode > VV_VAE_ROWS_ACC_TRUNC || out.rows.n <= 0 || out.rows.n > VV_VAE_MAX_ITEMS ||
         out.rows.seg[0].row0 != 0))
        return VV_ERR_INVALID_ARG;
    out.c = static_cast<vv::h16*>(C);
    out.ldc = ldc;
    out.bias = static_cast<const vv::h16*>(bias);
    vv::launch_vae_gemm<false, vv::kEpiRows>(static_cast<const vv::h16*>(A), lda, static_cast<const vv::h16*>(B), K, M, K,
                                            N, nullptr, nullptr, out, vv::as_stream(stream));
    return vv::launch_status();
}

vv_status_t vv_vae_f32_to_f16_dev(const float* in, void* out, int64_t n, void* stream) {
    if (!in || !out) return VV_ERR_NULL_PTR;
    if (n <= 0) return VV_OK;
    const int64_t blocks = (n + vv::kBlock - 1) / vv::kBlock;
    if (blocks > 0x7FFFFFFF) return VV_ERR_UNSUPPORTED;
    vv::vae_f32_to_f16<<<dim3((unsigned)blocks), vv::kBlock, 0, vv::as_stream(stream)>>>(in, static_cast<vv::h16*>(out), n);
    return vv::launch_status();
}

vv_status_t vv_gemm_fp16_nn_dev(const void* A, const void* B, void* C, int M, int K, int P, float alpha, float beta,
                                void* stream) {
    if (!A || !B || !C) return VV_ERR_NULL_PTR;
    if (M <= 0 || P <= 0) return VV_OK;
    if (K < 0) return VV_ERR_INVALID_ARG;
    vv::GemmOut out = {};
    out.c = static_cast<vv::h16*>(C);
    out.ldc = P;
    out.alpha = alpha;
    out.beta = beta;
    vv::launch_vae_gemm<true, vv::kEpiAlphaBeta>(static_cast<const vv::h16*>(A), K, static_cast<const vv::h16*>(B), P, M,
                                                 K, P, nullptr, nullptr, out, vv::as_stream(stream));
    return vv::launch_status();
}

void vv_gemm_cleanup(void) {}

}  // extern "C"
