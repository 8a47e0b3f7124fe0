// The older weight-only linear layers: FP16 activations against per-channel INT8,
// NF4 (bitsandbytes) or INT4 group-affine {scale, min} weights in their row-major
// stored forms (the formats of `--quant int8`, `--quant nf4` and a load-time
// repacked AWQ / GPTQ checkpoint when the accelerator layout is off).
//
//   wo_dequant  codes -> dense FP16 [N][K], one thread per eight weights, the
//               rounding rules of wonly.hpp (the same bits the small-M MFMA
//               kernel multiplies)
//   wo_gemv     1 <= M <= 8: a lane takes 16 bytes of codes per step (32 4-bit
//               or 16 int8 weights) and meets them with v_dot2_f32_f16. The
//               4-bit formats look a code byte up as a half2 in a 1 KB LDS
//               table (NF4: the code book rounded to FP16; INT4: the integers)
//               and apply the block's scale to the FP32 partial sum (INT4: and
//               the min to the sum of the activations); int8 codes become
//               exact FP16 integers by a byte permute and a packed subtract,
//               the row's FP32 scale applied once at the end.
//   larger M    9..64 rows go to the weight-streaming MFMA kernel of gemm.hip
//               (dequantised in registers, no scratch); beyond that, or where
//               that kernel declines, the weight is dequantised into the
//               caller's scratch and the FP16 GEMM runs on it: the same bits
//               either way.
#include "wonly.hpp"

// gemm.hip: one INT4 {scale, min} weight through the small-M MFMA kernel, or VV_ERR_UNSUPPORTED.
__attribute__((visibility("hidden")))
vv_status_t vv_skinny_int4_minmax(const void* A, const void* w, const void* scales, const void* mins, int gshift,
                                  void* y, int M, int N, int K, void* stream);

// gemm.hip: the same 9..64 rows where the small-M kernel declines, through the LDS-tiled kernel with the weight
// dequantised on its way in; VV_ERR_UNSUPPORTED outside what it covers.
__attribute__((visibility("hidden")))
vv_status_t vv_gemm_tile_weight_only(int format, const void* A, const void* w, const void* scales, const void* mins,
                                     int gshift, void* y, int M, int N, int K, void* stream);

namespace vv {
namespace {

typedef wo_u32x4 u32x4;

template <int kFmt>
__global__ __launch_bounds__(kBlock) void wo_dequant(WoSource src, u32x4* __restrict__ out, size_t n_slots, int K) {
    __shared__ float book[16];
    if constexpr (kFmt == kWoNf4) {
        if (threadIdx.x < 16) book[threadIdx.x] = kNf4Book[threadIdx.x];
        __syncthreads();
    }
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n_slots) return;
    const size_t per_row = (size_t)(K / 8);
    const size_t row = i / per_row;
    out[i] = wo_slot<kFmt>(src, book, row, K, (int)(i - row * per_row));
}

struct WoGemv {
    const u32x4* w;          // [N][K / kCols] 16-byte chunks of codes
    const void* scales;
    const h16* mins;
    const h16* bias;
    h16* y;
    int N, K, gshift;
};

template <int kFmt>
__device__ __forceinline__ uint32_t byte_table_entry(int b) {
    h16x2 v;
    if constexpr (kFmt == kWoNf4) v = h16x2{to_half(kNf4Book[b >> 4]), to_half(kNf4Book[b & 15])};
    else v = h16x2{(h16)(float)(b >> 4), (h16)(float)(b & 15)};
    return __builtin_bit_cast(uint32_t, v);
}

// kSplit waves share RW weight rows: wave p takes the rounds of 64 chunks p,
// p + kSplit, ...; lane l chunk l of the round, of each of its RW rows (the
// activation chunk is loaded once for all of them).
template <int kFmt, int MR, int kSplit, int RW>
__global__ __launch_bounds__(kBlock) void wo_gemv(const h16* __restrict__ x, WoGemv a, int M) {
    constexpr int kCols = kFmt == kWoInt8 ? 16 : 32;       // weights per 16-byte chunk
    constexpr int kRows = kWavesPerBlock / kSplit * RW;
    __shared__ uint32_t table[256];
    __shared__ float part[kWavesPerBlock][RW][MR];
    if constexpr (kFmt != kWoInt8) {
        table[threadIdx.x] = byte_table_entry<kFmt>((int)threadIdx.x);
        __syncthreads();
    }
    const int wave = wave_in_block(), lane = lane_id();
    const int set = wave / kSplit, piece = wave % kSplit;
    const int n0 = (int)blockIdx.x * kRows + set * RW;
    const int K = a.K, nchunks = K / kCols;
    size_t row[RW];
    const u32x4* wrow[RW];
#pragma unroll
    for (int r = 0; r < RW; ++r) {
        row[r] = (size_t)min(n0 + r, a.N - 1);
        wrow[r] = a.w + row[r] * nchunks;
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
        float sc[RW], mn[RW];
        h16x2 wv[RW][kCols / 2];                   // wv[r][p]: columns 2p, 2p + 1 of the chunk
#pragma unroll
        for (int r = 0; r < RW; ++r) {
            const u32x4 codes = __builtin_nontemporal_load(wrow[r] + c);
            sc[r] = 1.0f;
            mn[r] = 0.0f;
            if constexpr (kFmt == kWoNf4) {
                sc[r] = (float)static_cast<const h16*>(a.scales)[(row[r] * K + (size_t)c * kCols) >> 6];
            } else if constexpr (kFmt == kWoAwq) {
                const size_t g = row[r] * (size_t)(K >> a.gshift) + (size_t)((c * kCols) >> a.gshift);
                sc[r] = (float)static_cast<const h16*>(a.scales)[g];
                mn[r] = (float)a.mins[g];
            }
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                if constexpr (kFmt == kWoInt8) {
                    // byte -> 0x6400 | (q + 128) = 1152 + q as FP16; minus 1152 is exact
                    const uint32_t u = codes[t] ^ 0x80808080u;
                    const h16x2 off = {(h16)1152.0f, (h16)1152.0f};
                    wv[r][2 * t] = __builtin_bit_cast(h16x2, __builtin_amdgcn_perm(0x64646464u, u, 0x04010400u)) - off;
                    wv[r][2 * t + 1] = __builtin_bit_cast(h16x2, __builtin_amdgcn_perm(0x64646464u, u, 0x04030402u)) - off;
                } else {
#pragma unroll
                    for (int b = 0; b < 4; ++b)
                        wv[r][4 * t + b] = __builtin_bit_cast(h16x2, table[(codes[t] >> (8 * b)) & 0xFFu]);
                }
            }
        }
#pragma unroll
        for (int m = 0; m < MR; ++m) {
            if (m < M && live) {
                const u32x4* xr = reinterpret_cast<const u32x4*>(x + (size_t)m * K + (size_t)c * kCols);
                uint32_t xw[kCols / 2];
#pragma unroll
                for (int q = 0; q < kCols / 8; ++q) {
                    const u32x4 v = xr[q];
                    xw[4 * q] = v.x;
                    xw[4 * q + 1] = v.y;
                    xw[4 * q + 2] = v.z;
                    xw[4 * q + 3] = v.w;
                }
                float xs = 0.0f;
                if constexpr (kFmt == kWoAwq) {
                    const h16x2 ones = {(h16)1.0f, (h16)1.0f};
#pragma unroll
                    for (int p = 0; p < kCols / 2; ++p)
                        xs = __builtin_amdgcn_fdot2(ones, __builtin_bit_cast(h16x2, xw[p]), xs, false);
                }
#pragma unroll
                for (int r = 0; r < RW; ++r) {
                    float dot = kFmt == kWoInt8 ? acc[r][m] : 0.0f;
#pragma unroll
                    for (int p = 0; p < kCols / 2; ++p)
                        dot = __builtin_amdgcn_fdot2(wv[r][p], __builtin_bit_cast(h16x2, xw[p]), dot, false);
                    if constexpr (kFmt == kWoInt8) acc[r][m] = dot;
                    else if constexpr (kFmt == kWoNf4) acc[r][m] = __builtin_fmaf(sc[r], dot, acc[r][m]);
                    else acc[r][m] = __builtin_fmaf(sc[r], dot, __builtin_fmaf(mn[r], xs, acc[r][m]));
                }
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
        if (lane < RW * MR && m < M && n0 + r < a.N) {
            const int n = n0 + r;
            if constexpr (kFmt == kWoInt8) mine *= static_cast<const float*>(a.scales)[n];
            if (a.bias) mine += (float)a.bias[n];
            a.y[(size_t)m * a.N + n] = to_half(mine);
        }
    }
}

template <int kFmt, int MR, int kSplit, int RW>
void launch_gemv_cfg(const h16* x, const WoGemv& a, int M, hipStream_t st) {
    constexpr int kRows = kWavesPerBlock / kSplit * RW;
    wo_gemv<kFmt, MR, kSplit, RW><<<dim3((unsigned)((a.N + kRows - 1) / kRows)), kBlock, 0, st>>>(x, a, M);
}

template <int kFmt, int MR>
void launch_gemv_rows(const h16* x, const WoGemv& a, int M, hipStream_t st) {
    constexpr int kCols = kFmt == kWoInt8 ? 16 : 32;
    const int nchunks = a.K / kCols;
    // Thousands of waves in flight, and no wave with less than half a round of chunks; with rows to spare and short
    // rows, two or four rows per wave (each activation chunk loaded once for them).
    int split = 1, rw = 1;
    while (split < 4 && (long)a.N * split < 4096 && nchunks / (2 * split) >= kWave / 2) split *= 2;
    while (split == 1 && rw < 4 && a.N / (2 * rw) >= 8192 && nchunks * rw <= 256 && MR * rw * 2 <= 8) rw *= 2;
    if constexpr (MR <= 2) {
        if (rw == 4) return launch_gemv_cfg<kFmt, MR, 1, 4>(x, a, M, st);
    }
    if constexpr (MR <= 4) {
        if (rw >= 2) return launch_gemv_cfg<kFmt, MR, 1, 2>(x, a, M, st);
    }
    if (split == 1) launch_gemv_cfg<kFmt, MR, 1, 1>(x, a, M, st);
    else if (split == 2) launch_gemv_cfg<kFmt, MR, 2, 1>(x, a, M, st);
    else launch_gemv_cfg<kFmt, MR, 4, 1>(x, a, M, st);
}

template <int kFmt>
void launch_gemv(const h16* x, const WoGemv& a, int M, hipStream_t st) {
    if (M == 1) launch_gemv_rows<kFmt, 1>(x, a, M, st);
    else if (M == 2) launch_gemv_rows<kFmt, 2>(x, a, M, st);
    else if (M <= 4) launch_gemv_rows<kFmt, 4>(x, a, M, st);
    else launch_gemv_rows<kFmt, 8>(x, a, M, st);
}

int gshift_of(int group_size) {
    switch (group_size) {
        case 32: return 5;
        case 64: return 6;
        case 128: return 7;
        case 256: return 8;
        default: return -1;
    }
}

inline bool aligned4(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 3u) == 0; }
inline bool aligned2(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 1u) == 0; }
inline bool aligned8(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 7u) == 0; }

template <int kFmt>
vv_status_t dequant(const WoSource& src, void* out, size_t n_elements, int K, hipStream_t st) {
    const size_t slots = n_elements / 8;
    const size_t blocks = (slots + kBlock - 1) / kBlock;
    if (blocks > 0x7FFFFFFFu) return VV_ERR_UNSUPPORTED;
    wo_dequant<kFmt><<<dim3((unsigned)blocks), kBlock, 0, st>>>(src, static_cast<u32x4*>(out), slots, K);
    return launch_status();
}

// The GEMM behind the three entry points once M is past the one-row kernel:
// 9..64 rows through the small-M kernel where it serves, else dequantise into
// `temp` and multiply.
template <int kFmt>
vv_status_t gemm_via_fp16(const void* input, const WoSource& src, void* output, void* temp, int M, int N, int K,
                          void* stream) {
    if (M >= 9 && M <= 64) {
        vv_status_t s;
        if constexpr (kFmt == kWoAwq) {
            s = vv_skinny_int4_minmax(input, src.w, src.scales, src.mins, src.gshift, output, M, N, K, stream);
        } else {
            const vv_skinny_proj_t p = {src.w, src.scales, nullptr, output, N};
            s = vv_skinny_linear_dev(input, kFmt, &p, 1, M, K, 1.0f, stream);
        }
        if (s != VV_ERR_UNSUPPORTED) return s;
        s = vv_gemm_tile_weight_only(kFmt, input, src.w, src.scales, src.mins, src.gshift, output, M, N, K, stream);
        if (s != VV_ERR_UNSUPPORTED) return s;
    }
    if (!temp) return VV_ERR_NULL_PTR;
    if (!aligned16(temp)) return VV_ERR_UNSUPPORTED;
    const vv_status_t s = dequant<kFmt>(src, temp, (size_t)N * K, K, as_stream(stream));
    if (s != VV_OK) return s;
    return vv_gemm_fp16_dev(input, temp, output, M, N, K, 1.0f, 0.0f, stream);
}

}  // namespace
}  // namespace vv

extern "C" {

/* ── NF4 ─────────────────────────────────────────────────────────────────── */

vv_status_t vv_dequant_nf4_dev(const uint8_t* packed, const void* scales_fp16, void* output_fp16, int n_elements,
                               int block_size, void* stream) {
    if (!packed || !scales_fp16 || !output_fp16) return VV_ERR_NULL_PTR;
    if (n_elements <= 0 || block_size <= 0) return VV_ERR_INVALID_ARG;
    if (block_size != 64 || (n_elements & 7) != 0 || !vv::aligned4(packed) || !vv::aligned2(scales_fp16) ||
        !vv::aligned16(output_fp16))
        return VV_ERR_UNSUPPORTED;
    const vv::WoSource src = {packed, scales_fp16, nullptr, 0};
    // one flat row: element e of the weight is element e of "row 0"
    return vv::dequant<vv::kWoNf4>(src, output_fp16, (size_t)n_elements, n_elements, vv::as_stream(stream));
}

vv_status_t vv_nf4_gemv_dev(const void* x, const uint8_t* packed, const void* scales, const void* bias, void* y,
                            int N, int K, void* stream) {
    if (!x || !packed || !scales || !y) return VV_ERR_NULL_PTR;
    if (N <= 0) return VV_OK;
    if (K <= 0 || K % 32 != 0 || !vv::aligned16(x) || !vv::aligned16(packed) || !vv::aligned2(scales))
        return VV_ERR_UNSUPPORTED;
    const vv::WoGemv a = {reinterpret_cast<const vv::u32x4*>(packed), scales, nullptr,
                          static_cast<const vv::h16*>(bias), static_cast<vv::h16*>(y), N, K, 0};
    vv::launch_gemv<vv::kWoNf4>(static_cast<const vv::h16*>(x), a, 1, vv::as_stream(stream));
    return vv::launch_status();
}

vv_status_t vv_nf4_gemm_dev(const void* input_fp16, const uint8_t* weight_packed, const void* weight_scales_fp16,
                            void* output_fp16, void* temp_weight_fp16, int M, int N, int K, int block_size,
                            void* stream) {
    if (!input_fp16 || !weight_packed || !weight_scales_fp16 || !output_fp16) return VV_ERR_NULL_PTR;
    if (M <= 0 || N <= 0) return VV_OK;
    if (K <= 0 || block_size != 64 || K % 8 != 0 || !vv::aligned4(weight_packed) || !vv::aligned2(weight_scales_fp16))
        return VV_ERR_UNSUPPORTED;
    if (M <= 8 && K % 32 == 0 && vv::aligned16(input_fp16) && vv::aligned16(weight_packed)) {
        const vv::WoGemv a = {reinterpret_cast<const vv::u32x4*>(weight_packed), weight_scales_fp16, nullptr, nullptr,
                              static_cast<vv::h16*>(output_fp16), N, K, 0};
        vv::launch_gemv<vv::kWoNf4>(static_cast<const vv::h16*>(input_fp16), a, M, vv::as_stream(stream));
        return vv::launch_status();
    }
    const vv::WoSource src = {weight_packed, weight_scales_fp16, nullptr, 0};
    return vv::gemm_via_fp16<vv::kWoNf4>(input_fp16, src, output_fp16, temp_weight_fp16, M, N, K, stream);
}

/* ── INT4 group-affine, row-major {scale, min} form ──────────────────────── */

vv_status_t vv_dequant_awq_dev(const uint32_t* packed, const uint32_t* mins, const void* scales, void* output_fp16,
                               int N, int K, int group_size, void* stream) {
    if (!packed || !scales || !mins || !output_fp16) return VV_ERR_NULL_PTR;
    const int gs = vv::gshift_of(group_size);
    if (gs < 0 || K <= 0 || (K & 7) != 0 || K % group_size != 0 || !vv::aligned2(scales) || !vv::aligned2(mins) ||
        !vv::aligned16(output_fp16))
        return VV_ERR_UNSUPPORTED;
    if (N <= 0) return VV_OK;
    const vv::WoSource src = {packed, scales, mins, gs};
    return vv::dequant<vv::kWoAwq>(src, output_fp16, (size_t)N * K, K, vv::as_stream(stream));
}

vv_status_t vv_awq_gemv_dev(const void* x, const uint32_t* packed, const uint32_t* mins, const void* scales,
                            const void* bias, void* y, int N, int K, int group_size, void* stream) {
    if (!x || !packed || !scales || !mins || !y) return VV_ERR_NULL_PTR;
    const int gs = vv::gshift_of(group_size);
    if (gs < 0 || K <= 0 || K % 32 != 0 || K % group_size != 0 || !vv::aligned16(x) || !vv::aligned16(packed) ||
        !vv::aligned2(scales) || !vv::aligned2(mins))
        return VV_ERR_UNSUPPORTED;
    if (N <= 0) return VV_OK;
    const vv::WoGemv a = {reinterpret_cast<const vv::u32x4*>(packed), scales, reinterpret_cast<const vv::h16*>(mins),
                          static_cast<const vv::h16*>(bias), static_cast<vv::h16*>(y), N, K, gs};
    vv::launch_gemv<vv::kWoAwq>(static_cast<const vv::h16*>(x), a, 1, vv::as_stream(stream));
    return vv::launch_status();
}

vv_status_t vv_awq_gemm_dev(const void* input_fp16, const uint32_t* packed, const uint32_t* mins, const void* scales,
                            void* output_fp16, void* temp_weight_fp16, int M, int N, int K, int group_size,
                            void* stream) {
    if (!input_fp16 || !packed || !scales || !mins || !output_fp16) return VV_ERR_NULL_PTR;
    const int gs = vv::gshift_of(group_size);
    if (gs < 0 || K <= 0 || (K & 7) != 0 || K % group_size != 0 || !vv::aligned2(scales) || !vv::aligned2(mins))
        return VV_ERR_UNSUPPORTED;
    if (M <= 0 || N <= 0) return VV_OK;
    if (M <= 8 && K % 32 == 0 && vv::aligned16(input_fp16) && vv::aligned16(packed)) {
        const vv::WoGemv a = {reinterpret_cast<const vv::u32x4*>(packed), scales, reinterpret_cast<const vv::h16*>(mins),
                              nullptr, static_cast<vv::h16*>(output_fp16), N, K, gs};
        vv::launch_gemv<vv::kWoAwq>(static_cast<const vv::h16*>(input_fp16), a, M, vv::as_stream(stream));
        return vv::launch_status();
    }
    const vv::WoSource src = {packed, scales, mins, gs};
    return vv::gemm_via_fp16<vv::kWoAwq>(input_fp16, src, output_fp16, temp_weight_fp16, M, N, K, stream);
}

/* ── per-channel INT8 ────────────────────────────────────────────────────── */

vv_status_t vv_dequant_int8_dev(const int8_t* q, const float* scales, void* output_fp16, int N, int K, void* stream) {
    if (!q || !scales || !output_fp16) return VV_ERR_NULL_PTR;
    if (N <= 0 || K <= 0 || (K & 15) != 0 || !vv::aligned8(q) || !vv::aligned4(scales) || !vv::aligned16(output_fp16))
        return VV_ERR_UNSUPPORTED;
    const vv::WoSource src = {q, scales, nullptr, 0};
    return vv::dequant<vv::kWoInt8>(src, output_fp16, (size_t)N * K, K, vv::as_stream(stream));
}

vv_status_t vv_int8_gemv_dev(const void* x, const int8_t* q, const float* scales, const void* bias, void* y, int N,
                             int K, void* stream) {
    if (!x || !q || !scales || !y) return VV_ERR_NULL_PTR;
    if (N <= 0 || K <= 0 || (K & 15) != 0 || !vv::aligned16(x) || !vv::aligned16(q) || !vv::aligned4(scales))
        return VV_ERR_UNSUPPORTED;
    const vv::WoGemv a = {reinterpret_cast<const vv::u32x4*>(q), scales, nullptr, static_cast<const vv::h16*>(bias),
                          static_cast<vv::h16*>(y), N, K, 0};
    vv::launch_gemv<vv::kWoInt8>(static_cast<const vv::h16*>(x), a, 1, vv::as_stream(stream));
    return vv::launch_status();
}

vv_status_t vv_int8_gemm_dev(const void* input_fp16, const int8_t* q, const float* scales, void* output_fp16,
                             void* temp_weight_fp16, int M, int N, int K, void* stream) {
    if (!input_fp16 || !q || !scales || !output_fp16) return VV_ERR_NULL_PTR;
    if (M <= 0 || N <= 0 || K <= 0 || (K & 15) != 0 || !vv::aligned8(q) || !vv::aligned4(scales))
        return VV_ERR_UNSUPPORTED;
    if (M <= 8 && vv::aligned16(input_fp16) && vv::aligned16(q)) {
        const vv::WoGemv a = {reinterpret_cast<const vv::u32x4*>(q), scales, nullptr, nullptr,
                              static_cast<vv::h16*>(output_fp16), N, K, 0};
        vv::launch_gemv<vv::kWoInt8>(static_cast<const vv::h16*>(input_fp16), a, M, vv::as_stream(stream));
        return vv::launch_status();
    }
    const vv::WoSource src = {q, scales, nullptr, 0};
    return vv::gemm_via_fp16<vv::kWoInt8>(input_fp16, src, output_fp16, temp_weight_fp16, M, N, K, stream);
}

}  // extern "C"
