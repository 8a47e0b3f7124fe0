// Flat elementwise kernels: SwiGLU, residual add, bias add, FP32 <-> FP16.
//
// Each is a single pass over contiguous FP16 data, bound by HBM bandwidth. A
// thread moves kUnroll 16-byte chunks per input, all of its loads issued before
// the first use, the chunks of one instruction contiguous across the wave
// (64 lanes x 16 B = 1 KiB per load instruction). Every thread reads all of its
// chunks before it writes any of them and no other thread touches those
// chunks, so an output that aliases an input exactly (out == gate, the way the
// decoder calls SwiGLU) is safe. Unaligned pointers take a 2-byte kernel.
#include "vv_common.hpp"

namespace vv {
namespace {

constexpr int kUnroll = 4;                       // chunks per thread per input
constexpr int kChunksPerBlock = kBlock * kUnroll;

// silu(g) * u in the oracle's association, (g / (1 + e^-g)) * u, with the
// hardware exponential and reciprocal: exp2(-g * log2 e) and rcp are each
// accurate to about 1 ulp of FP32, three orders below the FP16 rounding of the
// result. Large |g| needs no special case: e^-g -> inf gives rcp -> 0 and
// g * 0 = -0 (the oracle's -65504 / inf), e^-g -> 0 gives g itself.
__device__ __forceinline__ float swiglu1(float g, float u) {
    const float e = __builtin_amdgcn_exp2f(g * -1.44269504088896340736f);
    const float silu = g * __builtin_amdgcn_rcpf(1.0f + e);
    return silu * u;
}

enum EwOp : int { kSwiglu = 0, kResidual = 1 };

template <int kOp>
__device__ __forceinline__ Chunk apply2(const Chunk& a, const Chunk& b) {
    const f32x8 x = unpack(a), y = unpack(b);
    f32x8 r;
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = (kOp == kSwiglu) ? swiglu1(x[i], y[i]) : (x[i] + y[i]);
    return pack(r);
}

template <int kOp>
__device__ __forceinline__ h16 apply2(h16 a, h16 b) {
    return to_half((kOp == kSwiglu) ? swiglu1((float)a, (float)b) : ((float)a + (float)b));
}

// out[i] = op(a[i], b[i]) over nchunks chunks, then the (< 8) trailing halves.
template <int kOp, bool kStream>
__global__ __launch_bounds__(kBlock) void binary_chunks(const Chunk* a, const Chunk* b,
                                                        Chunk* out, size_t nchunks,
                                                        int tail_halves) {
    const size_t base = (size_t)blockIdx.x * kChunksPerBlock + threadIdx.x;
    Chunk va[kUnroll], vb[kUnroll];
    if (base + (size_t)(kUnroll - 1) * kBlock < nchunks) {
#pragma unroll
        for (int j = 0; j < kUnroll; ++j) {
            va[j] = load_chunk_as<kStream>(a + base + (size_t)j * kBlock);
            vb[j] = load_chunk_as<kStream>(b + base + (size_t)j * kBlock);
        }
#pragma unroll
        for (int j = 0; j < kUnroll; ++j)
            store_chunk_as<kStream>(out + base + (size_t)j * kBlock, apply2<kOp>(va[j], vb[j]));
    } else {
#pragma unroll
        for (int j = 0; j < kUnroll; ++j) {
            const size_t c = base + (size_t)j * kBlock;
            if (c < nchunks) { va[j] = load_chunk(a + c); vb[j] = load_chunk(b + c); }
        }
#pragma unroll
        for (int j = 0; j < kUnroll; ++j) {
            const size_t c = base + (size_t)j * kBlock;
            if (c < nchunks) store_chunk(out + c, apply2<kOp>(va[j], vb[j]));
        }
    }
    if (tail_halves > 0 && blockIdx.x == 0 && (int)threadIdx.x < tail_halves) {
        const h16* ta = reinterpret_cast<const h16*>(a + nchunks);
        const h16* tb = reinterpret_cast<const h16*>(b + nchunks);
        h16* to = reinterpret_cast<h16*>(out + nchunks);
        to[threadIdx.x] = apply2<kOp>(ta[threadIdx.x], tb[threadIdx.x]);
    }
}

template <int kOp>
__global__ __launch_bounds__(kBlock) void binary_halves(const h16* a, const h16* b, h16* out,
                                                        size_t n) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) out[i] = apply2<kOp>(a[i], b[i]);
}

template <int kOp>
vv_status_t launch_binary(const void* a, const void* b, void* out, size_t n, hipStream_t st) {
    if (n == 0) return VV_OK;
    if (aligned16(a) && aligned16(b) && aligned16(out)) {
        const size_t nchunks = n / 8;
        const int tail = (int)(n % 8);
        const size_t blocks = nchunks ? (nchunks + kChunksPerBlock - 1) / kChunksPerBlock : 1;
        if (use_streaming(3u * n * 2u))
            binary_chunks<kOp, true><<<dim3((unsigned)blocks), kBlock, 0, st>>>(
                static_cast<const Chunk*>(a), static_cast<const Chunk*>(b),
                static_cast<Chunk*>(out), nchunks, tail);
        else
            binary_chunks<kOp, false><<<dim3((unsigned)blocks), kBlock, 0, st>>>(
                static_cast<const Chunk*>(a), static_cast<const Chunk*>(b),
                static_cast<Chunk*>(out), nchunks, tail);
    } else {
        const size_t blocks = (n + kBlock - 1) / kBlock;
        binary_halves<kOp><<<dim3((unsigned)blocks), kBlock, 0, st>>>(
            static_cast<const h16*>(a), static_cast<const h16*>(b), static_cast<h16*>(out), n);
    }
    return launch_status();
}

// gate and up are the two halves of each [2*inter] row. One workgroup column
// per row (blockIdx.y), chunks of the row spread over blockIdx.x.
__global__ __launch_bounds__(kBlock) void swiglu_fused_chunks(const Chunk* gate_up, Chunk* out,
                                                              int inter_chunks) {
    const size_t row = blockIdx.y;
    const Chunk* g = gate_up + row * 2u * (size_t)inter_chunks;
    const Chunk* u = g + inter_chunks;
    Chunk* o = out + row * (size_t)inter_chunks;
    const int base = (int)blockIdx.x * kChunksPerBlock + (int)threadIdx.x;
    Chunk vg[kUnroll], vu[kUnroll];
#pragma unroll
    for (int j = 0; j < kUnroll; ++j) {
        const int c = base + j * kBlock;
        if (c < inter_chunks) { vg[j] = load_chunk(g + c); vu[j] = load_chunk(u + c); }
    }
#pragma unroll
    for (int j = 0; j < kUnroll; ++j) {
        const int c = base + j * kBlock;
        if (c < inter_chunks) store_chunk(o + c, apply2<kSwiglu>(vg[j], vu[j]));
    }
}

__global__ __launch_bounds__(kBlock) void swiglu_fused_halves(const h16* gate_up, h16* out,
                                                              int inter) {
    const size_t row = blockIdx.y;
    const int c = (int)blockIdx.x * kBlock + (int)threadIdx.x;
    if (c >= inter) return;
    const h16* g = gate_up + row * 2u * (size_t)inter;
    out[row * (size_t)inter + c] = apply2<kSwiglu>(g[c], g[inter + c]);
}

// out[m, :] += bias[:]. Chunked form: a row is n_chunks chunks, the bias chunk
// index is the chunk's column, found with one 64-bit modulo per chunk.
__global__ __launch_bounds__(kBlock) void bias_add_chunks(Chunk* out, const Chunk* __restrict__ bias,
                                                          size_t total_chunks, int row_chunks) {
    const size_t base = (size_t)blockIdx.x * kChunksPerBlock + threadIdx.x;
    Chunk v[kUnroll];
#pragma unroll
    for (int j = 0; j < kUnroll; ++j) {
        const size_t c = base + (size_t)j * kBlock;
        if (c < total_chunks) v[j] = load_chunk(out + c);
    }
#pragma unroll
    for (int j = 0; j < kUnroll; ++j) {
        const size_t c = base + (size_t)j * kBlock;
        if (c < total_chunks) {
            const Chunk bv = load_chunk(bias + (c % (size_t)row_chunks));
            store_chunk(out + c, apply2<kResidual>(v[j], bv));
        }
    }
}

__global__ __launch_bounds__(kBlock) void bias_add_halves(h16* out, const h16* __restrict__ bias,
                                                          size_t total, int n) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < total) out[i] = to_half((float)out[i] + (float)bias[i % (size_t)n]);
}

__global__ __launch_bounds__(kBlock) void f32_to_f16(const float* __restrict__ in,
                                                     h16* __restrict__ out, size_t n) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) out[i] = to_half(in[i]);
}

__global__ __launch_bounds__(kBlock) void f16_to_f32(const h16* __restrict__ in,
                                                     float* __restrict__ out, size_t n) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) out[i] = (float)in[i];
}

}  // namespace
}  // namespace vv

extern "C" {

vv_status_t vv_swiglu_dev(const void* gate, const void* up, void* output, int n_elements,
                          void* stream) {
    if (!gate || !up || !output) return VV_ERR_NULL_PTR;
    if (n_elements <= 0) return VV_OK;
    return vv::launch_binary<vv::kSwiglu>(gate, up, output, (size_t)n_elements,
                                          vv::as_stream(stream));
}

vv_status_t vv_residual_add_dev(void* x, const void* y, int total, void* stream) {
    if (!x || !y) return VV_ERR_NULL_PTR;
    if (total <= 0) return VV_OK;
    return vv::launch_binary<vv::kResidual>(x, y, x, (size_t)total, vv::as_stream(stream));
}

vv_status_t vv_swiglu_fused_dev(const void* gate_up, void* output, int rows, int inter,
                                void* stream) {
    if (!gate_up || !output) return VV_ERR_NULL_PTR;
    if (rows <= 0 || inter <= 0) return VV_OK;
    hipStream_t st = vv::as_stream(stream);
    if (inter % 8 == 0 && vv::aligned16(gate_up) && vv::aligned16(output)) {
        const int ic = inter / 8;
        const dim3 grid((unsigned)((ic + vv::kChunksPerBlock - 1) / vv::kChunksPerBlock),
                        (unsigned)rows);
        vv::swiglu_fused_chunks<<<grid, vv::kBlock, 0, st>>>(
            static_cast<const vv::Chunk*>(gate_up), static_cast<vv::Chunk*>(output), ic);
    } else {
        const dim3 grid((unsigned)((inter + vv::kBlock - 1) / vv::kBlock), (unsigned)rows);
        vv::swiglu_fused_halves<<<grid, vv::kBlock, 0, st>>>(
            static_cast<const vv::h16*>(gate_up), static_cast<vv::h16*>(output), inter);
    }
    return vv::launch_status();
}

vv_status_t vv_bias_add_dev(void* output, const void* bias, int M, int N, void* stream) {
    if (!output || !bias) return VV_ERR_NULL_PTR;
    if (M <= 0 || N <= 0) return VV_OK;
    hipStream_t st = vv::as_stream(stream);
    const size_t total = (size_t)M * (size_t)N;
    if (N % 8 == 0 && vv::aligned16(output) && vv::aligned16(bias)) {
        const size_t chunks = total / 8;
        const size_t blocks = (chunks + vv::kChunksPerBlock - 1) / vv::kChunksPerBlock;
        vv::bias_add_chunks<<<dim3((unsigned)blocks), vv::kBlock, 0, st>>>(
            static_cast<vv::Chunk*>(output), static_cast<const vv::Chunk*>(bias), chunks, N / 8);
    } else {
        const size_t blocks = (total + vv::kBlock - 1) / vv::kBlock;
        vv::bias_add_halves<<<dim3((unsigned)blocks), vv::kBlock, 0, st>>>(
            static_cast<vv::h16*>(output), static_cast<const vv::h16*>(bias), total, N);
    }
    return vv::launch_status();
}

vv_status_t vv_fp32_to_fp16_dev(const void* in_fp32, void* out_fp16, int n, void* stream) {
    if (!in_fp32 || !out_fp16) return VV_ERR_NULL_PTR;
    if (n <= 0) return VV_OK;
    const size_t blocks = ((size_t)n + vv::kBlock - 1) / vv::kBlock;
    vv::f32_to_f16<<<dim3((unsigned)blocks), vv::kBlock, 0, vv::as_stream(stream)>>>(
        static_cast<const float*>(in_fp32), static_cast<vv::h16*>(out_fp16), (size_t)n);
    return vv::launch_status();
}

vv_status_t vv_fp16_to_fp32_dev(const void* in_fp16, void* out_fp32, int n, void* stream) {
    if (!in_fp16 || !out_fp32) return VV_ERR_NULL_PTR;
    if (n <= 0) return VV_OK;
    const size_t blocks = ((size_t)n + vv::kBlock - 1) / vv::kBlock;
    vv::f16_to_f32<<<dim3((unsigned)blocks), vv::kBlock, 0, vv::as_stream(stream)>>>(
        static_cast<const vv::h16*>(in_fp16), static_cast<float*>(out_fp32), (size_t)n);
    return vv::launch_status();
}

}  // extern "C"
