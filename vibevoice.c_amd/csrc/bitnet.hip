// BitNet's integer layers: ternary (I2_S codes, one FP32 scale per tensor) and
// int8 weights against per-token int8 activations. Integer sums are exact, so
// the int32 accumulators equal the CPU's whatever the order they are added in;
// the FP32 steps after them are taken one rounding at a time, in the order the
// interface states, so the FP32 bits equal the CPU's too.
//
//   bn_act_quant  one workgroup per row: max |x|, s = (float)(127 / max(amax,
//                 1e-5)) in double, q = the integer that fma(x, s, 1.5 * 2^23)
//                 carries in its mantissa (the product is never rounded on its
//                 own), clamped to [-128, 127]; the row sum of q beside it
//   bn_gemm       16 or 32 weight rows per workgroup against 16 or 32 activation
//                 rows (grid.y walks M), K split over the eight waves, operands
//                 from global memory straight into v_mfma_i32_16x16x64_i8 with
//                 16-byte loads. Sixteen consecutive columns of a 128-block are
//                 one bit plane of sixteen consecutive code bytes, so a lane's
//                 16-byte load of codes gives its operands of both 64-column
//                 steps of the block by a shift and a mask. Codes stay 0..2; the
//                 row sum of the activations is subtracted once at the end:
//                 sum (c - 1) q = sum c q - sum q.
//   bn_naive      int8 x int8 when K is not a multiple of 16 or an operand is
//                 off 16 bytes: one thread per output
#include <float.h>

#include "vv_common.hpp"

namespace vv {
namespace {

typedef int i32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ int wave_sum_int(int v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

// ── activation quantiser ────────────────────────────────────────────────────

template <bool kF16>
__device__ __forceinline__ float bn_load(const void* x, size_t i) {
    if constexpr (kF16) return (float)static_cast<const h16*>(x)[i];
    else return static_cast<const float*>(x)[i];
}

template <bool kF16>
__global__ __launch_bounds__(kBlock) void bn_act_quant(const void* __restrict__ x, int K, int8_t* __restrict__ q,
                                                       float* __restrict__ scale, int32_t* __restrict__ sum) {
    __shared__ float wave_amax[kWavesPerBlock];
    __shared__ int wave_total[kWavesPerBlock];
    __shared__ float row_scale;
    const size_t base = (size_t)blockIdx.x * K;
    const int wave = wave_in_block(), lane = lane_id();
    float amax = 0.0f;
    for (int k = (int)threadIdx.x; k < K; k += kBlock) amax = fmaxf(amax, fabsf(bn_load<kF16>(x, base + k)));
    amax = wave_max(amax);
    if (lane == 0) wave_amax[wave] = amax;
    __syncthreads();
    if (threadIdx.x == 0) {
        float mx = 0.0f;
#pragma unroll
        for (int w = 0; w < kWavesPerBlock; ++w) mx = fmaxf(mx, wave_amax[w]);
        const double d = mx > 0.00001 ? (double)mx : 0.00001;
        row_scale = (float)(127.0 / d);
    }
    __syncthreads();
    const float s = row_scale;
    int total = 0;
    for (int k = (int)threadIdx.x; k < K; k += kBlock) {
        const float t = __builtin_fmaf(bn_load<kF16>(x, base + k), s, 12582912.0f);
        int v = (__builtin_bit_cast(int, t) & 0x007fffff) - 0x00400000;
        v = v > 127 ? 127 : (v < -128 ? -128 : v);
        q[base + k] = (int8_t)v;
        total += v;
    }
    total = wave_sum_int(total);
    if (lane == 0) wave_total[wave] = total;
    __syncthreads();
    if (threadIdx.x == 0) {
        int t = 0;
#pragma unroll
        for (int w = 0; w < kWavesPerBlock; ++w) t += wave_total[w];
        scale[blockIdx.x] = s;
        if (sum) sum[blockIdx.x] = t;
    }
}

// ── the shared epilogue ─────────────────────────────────────────────────────

struct BnOut {
    const int32_t* xsum;     // ternary: row sums of the activations, subtracted
    const float* x_scale;    // ternary: per-row multiplier
    const float* a_scale;    // int8: one multiplier, in device memory
    float w_scale;
    const float* bias;
    int32_t* acc;
    void* y;
    float* absmax;           // int8: max |y| folded in (must start at 0)
    int y_f16, tern;
    int M, N;
};

// One output: returns |y| (0 when no y is asked for). Every FP32 operation
// rounds on its own.
__device__ __forceinline__ float bn_finish(const BnOut& o, int m, int n, int v) {
#pragma clang fp contract(off)
    if (o.tern) v -= o.xsum[m];
    const size_t at = (size_t)m * o.N + n;
    if (o.acc) o.acc[at] = v;
    if (!o.y) return 0.0f;
    float r;
    if (o.tern) {
        r = (float)v / o.x_scale[m];
        r = r * o.w_scale;
    } else {
        const float d = o.w_scale / *o.a_scale;
        r = (float)v * d;
    }
    if (o.bias) r = r + o.bias[n];
    if (o.y_f16) static_cast<h16*>(o.y)[at] = to_half(r);
    else static_cast<float*>(o.y)[at] = r;
    return fabsf(r);
}

// Non-negative floats order like their bit patterns.
__device__ __forceinline__ void bn_fold_absmax(float* absmax, float v) {
    v = wave_max(v);
    if (lane_id() == 0 && v > 0.0f) atomicMax(reinterpret_cast<int*>(absmax), __builtin_bit_cast(int, v));
}

// ── the product ─────────────────────────────────────────────────────────────

constexpr int kBnWaves = 8;

// kRG groups of sixteen weight rows against kMT tiles of sixteen activation rows per workgroup; a wave takes every
// eighth 128-column block (two MFMA steps of 64 columns, a lane's share of a step being 16 consecutive columns).
template <bool kTern, int kMT, int kRG>
__global__ __launch_bounds__(kBnWaves * kWave) void bn_gemm(const int8_t* __restrict__ a, const void* __restrict__ w,
                                                            BnOut out, int K) {
    __shared__ i32x4 part[kBnWaves][kMT * kRG][kWave];
    const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r16 = lane & 15, ks = lane >> 4;
    const int n0 = (int)blockIdx.x * (16 * kRG), m0 = (int)blockIdx.y * (16 * kMT);
    const int kchunks = K / 16, nblocks = (kchunks + 7) / 8;
    size_t wrow[kRG];
#pragma unroll
    for (int g = 0; g < kRG; ++g) wrow[g] = (size_t)min(n0 + 16 * g + r16, out.N - 1);
    const i32x4* xrow[kMT];
#pragma unroll
    for (int t = 0; t < kMT; ++t)
        xrow[t] = reinterpret_cast<const i32x4*>(a + (size_t)min(m0 + 16 * t + r16, out.M - 1) * K);
    const i32x4 zero = {0, 0, 0, 0};
    i32x4 acc[kMT][kRG];
#pragma unroll
    for (int t = 0; t < kMT; ++t)
#pragma unroll
        for (int g = 0; g < kRG; ++g) acc[t][g] = zero;

    for (int b = wave; b < nblocks; b += kBnWaves) {
        i32x4 wv[kRG][2], xv[kMT][2];
        // activations: step s of the block is chunks 4 s .. 4 s + 3, this lane's being 4 s + ks
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            const int c = b * 8 + 4 * s + ks;
            const bool live = c < kchunks;
#pragma unroll
            for (int t = 0; t < kMT; ++t) xv[t][s] = live ? xrow[t][live ? c : 0] : zero;
        }
        if constexpr (kTern) {
            // Columns 16 j .. 16 j + 15 of a block (j = 4 s + ks) are bit plane j / 2 = 2 s + ks / 2 of code bytes
            // 16 (j % 2) .. + 15 = 16 (ks % 2) ..: one 16-byte load of codes serves both steps (K % 128 == 0).
#pragma unroll
            for (int g = 0; g < kRG; ++g) {
                const i32x4 codes = __builtin_nontemporal_load(
                    reinterpret_cast<const i32x4*>(static_cast<const uint8_t*>(w) + wrow[g] * (size_t)(K / 4)) + b * 2 +
                    (ks & 1));
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    const int shift = 6 - 2 * (2 * s + (ks >> 1));
#pragma unroll
                    for (int e = 0; e < 4; ++e) wv[g][s][e] = (int)(((uint32_t)codes[e] >> shift) & 0x03030303u);
                }
            }
        } else {
#pragma unroll
            for (int g = 0; g < kRG; ++g)
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    const int c = b * 8 + 4 * s + ks;
                    const bool live = c < kchunks;
                    wv[g][s] = live ? __builtin_nontemporal_load(
                                          reinterpret_cast<const i32x4*>(static_cast<const int8_t*>(w) + wrow[g] * K) +
                                          (live ? c : 0))
                                    : zero;
                }
        }
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int t = 0; t < kMT; ++t)
#pragma unroll
                for (int g = 0; g < kRG; ++g)
                    acc[t][g] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wv[g][s], xv[t][s], acc[t][g], 0, 0, 0);
    }
#pragma unroll
    for (int t = 0; t < kMT; ++t)
#pragma unroll
        for (int g = 0; g < kRG; ++g) part[wave][t * kRG + g][lane] = acc[t][g];
    __syncthreads();

    // register r of lane l: column n0 + 16 g + 4 (l / 16) + r of row m0 + 16 t + l % 16
    float amax = 0.0f;
    constexpr int kTiles = kMT * kRG;
    for (int tile = wave; tile < kTiles; tile += kBnWaves) {
        i32x4 sum = part[0][tile][lane];
#pragma unroll
        for (int p = 1; p < kBnWaves; ++p) sum += part[p][tile][lane];
        const int t = tile / kRG, g = tile % kRG;
        const int m = m0 + 16 * t + r16, n = n0 + 16 * g + 4 * ks;
        if (m < out.M) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (n + r < out.N) amax = fmaxf(amax, bn_finish(out, m, n + r, sum[r]));
        }
    }
    if (!kTern && out.absmax && out.y && wave < kTiles) bn_fold_absmax(out.absmax, amax);
}

__global__ __launch_bounds__(kBlock) void bn_naive(const int8_t* __restrict__ a, const int8_t* __restrict__ w, BnOut out,
                                                   int K) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    const bool live = i < (size_t)out.M * out.N;
    float amax = 0.0f;
    if (live) {
        const int m = (int)(i / out.N), n = (int)(i % out.N);
        const int8_t* ar = a + (size_t)m * K;
        const int8_t* wr = w + (size_t)n * K;
        int s = 0;
        for (int k = 0; k < K; ++k) s += (int)wr[k] * (int)ar[k];
        amax = bn_finish(out, m, n, s);
    }
    if (out.absmax && out.y) bn_fold_absmax(out.absmax, amax);
}

template <bool kTern>
void launch_bn_gemm(const int8_t* a, const void* w, const BnOut& out, int K, hipStream_t st) {
    constexpr int kThreads = kBnWaves * kWave;
    if (out.M <= 16) {          // decode and a few rows: sixteen weight rows per workgroup, the most workgroups
        const dim3 grid((unsigned)((out.N + 15) / 16), 1);
        bn_gemm<kTern, 1, 1><<<grid, kThreads, 0, st>>>(a, w, out, K);
    } else {                    // 32 x 32 outputs per workgroup: each operand register feeds two products
        const dim3 grid((unsigned)((out.N + 31) / 32), (unsigned)((out.M + 31) / 32));
        bn_gemm<kTern, 2, 2><<<grid, kThreads, 0, st>>>(a, w, out, K);
    }
}

// The requantiser and the int8 tied head are not built in this backend: their entry points answer
// VV_ERR_UNSUPPORTED.
constexpr int kHeadRows = 128;      // weight rows per partial winner: sizes vv_i8_head_argmax_scratch_bytes

}  // namespace
}  // namespace vv

extern "C" {

vv_status_t vv_act_quant_i8_dev(const void* x, int x_f16, int M, int K, int8_t* q, float* scale, int32_t* sum,
                                void* stream) {
    if (!x || !q || !scale) return VV_ERR_NULL_PTR;
    if (M <= 0 || K <= 0) return VV_ERR_INVALID_ARG;
    hipStream_t st = vv::as_stream(stream);
    if (x_f16) vv::bn_act_quant<true><<<dim3((unsigned)M), vv::kBlock, 0, st>>>(x, K, q, scale, sum);
    else vv::bn_act_quant<false><<<dim3((unsigned)M), vv::kBlock, 0, st>>>(x, K, q, scale, sum);
    return vv::launch_status();
}

vv_status_t vv_ternary_gemm_dev(const int8_t* q, const int32_t* xsum, const float* x_scale, const uint8_t* codes,
                                float w_scale, const float* bias, int32_t* acc, void* y, int y_f16, int M, int N,
                                int K, void* stream) {
    if (!q || !xsum || !codes) return VV_ERR_NULL_PTR;
    if (y && !x_scale) return VV_ERR_NULL_PTR;
    if (M <= 0 || N <= 0 || K <= 0 || K % 128) return VV_ERR_INVALID_ARG;
    if (!vv::aligned16(q) || !vv::aligned16(codes)) return VV_ERR_UNSUPPORTED;      // 16-byte operand loads
    vv::BnOut out = {};
    out.xsum = xsum;
    out.x_scale = x_scale;
    out.w_scale = w_scale;
    out.bias = bias;
    out.acc = acc;
    out.y = y;
    out.y_f16 = y_f16;
    out.tern = 1;
    out.M = M;
    out.N = N;
    vv::launch_bn_gemm<true>(q, codes, out, K, vv::as_stream(stream));
    return vv::launch_status();
}

vv_status_t vv_i8_gemm_dev(const int8_t* a, const float* a_scale, const int8_t* w, float w_scale, const float* bias,
                           int32_t* acc, float* y, float* absmax, int M, int N, int K, void* stream) {
    if (!a || !w) return VV_ERR_NULL_PTR;
    if (y && !a_scale) return VV_ERR_NULL_PTR;
    if (M <= 0 || N <= 0 || K <= 0) return VV_ERR_INVALID_ARG;
    vv::BnOut out = {};
    out.a_scale = a_scale;
    out.w_scale = w_scale;
    out.bias = bias;
    out.acc = acc;
    out.y = y;
    out.absmax = y ? absmax : nullptr;
    out.M = M;
    out.N = N;
    hipStream_t st = vv::as_stream(stream);
    if (K % 16 == 0 && vv::aligned16(a) && vv::aligned16(w)) {
        vv::launch_bn_gemm<false>(a, w, out, K, st);
    } else {
        const size_t blocks = ((size_t)M * N + vv::kBlock - 1) / vv::kBlock;
        if (blocks > 0x7FFFFFFFu) return VV_ERR_UNSUPPORTED;
        vv::bn_naive<<<dim3((unsigned)blocks), vv::kBlock, 0, st>>>(a, w, out, K);
    }
    return vv::launch_status();
}

vv_status_t vv_i8s_requant_dev(const float* y, int64_t n, const float* absmax, int relu, int8_t* q, float* out_scale,
                               void* stream) {
    (void)y; (void)n; (void)absmax; (void)relu; (void)q; (void)out_scale; (void)stream;
    return VV_ERR_UNSUPPORTED;      // not built in this backend: nothing is launched
}

size_t vv_i8_head_argmax_scratch_bytes(int V) {
    if (V <= 0) return 0;
    const size_t nb = ((size_t)V + vv::kHeadRows - 1) / vv::kHeadRows;
    return nb * (sizeof(float) + sizeof(int));
}

vv_status_t vv_i8_head_argmax_dev(const int8_t* q, const float* scale, const int8_t* w, const float* w_scale, int V,
                                  int K, int32_t* token, float* value, void* scratch, void* stream) {
    (void)q; (void)scale; (void)w; (void)w_scale; (void)V; (void)K; (void)token; (void)value; (void)scratch;
    (void)stream;
    return VV_ERR_UNSUPPORTED;      // not built in this backend: nothing is launched
}

}  // extern "C"
