// Flat elementwise kernels: SwiGLU, residual add, bias add, FP32 <-> FP16.
//
// Each is a single pass over contiguous FP16 data, bound by HBM bandwidth. A
// thread moves ONE 16-byte chunk per input and a workgroup is ONE wave: the
// chunks of a load instruction are contiguous across the wave (64 lanes x 16 B
// = 1 KiB), and the grid is as many light, short-lived waves as there are KiB.
// Measured for SwiGLU at T = 14449 (1.64 GB per launch): 1 chunk/thread in
// 64-thread workgroups 84.3 % of the HBM peak, in 256-thread workgroups 82.7 %,
// 4 chunks/thread in 256-thread workgroups 75.9-79.6 %. Every thread reads its
// chunk before it writes it and no other thread touches that chunk, so an
// output that aliases an input exactly (out == gate, the way the decoder calls
// SwiGLU) is safe. Unaligned pointers take a 2-byte kernel.
#include "row_math.hpp"

namespace vv {
namespace {

constexpr int kEwBlock = kWave;                  // one wave per workgroup

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
__global__ __launch_bounds__(kEwBlock) void binary_chunks(const Chunk* a, const Chunk* b,
                                                          Chunk* out, size_t nchunks,
                                                          int tail_halves) {
    const size_t c = (size_t)blockIdx.x * kEwBlock + threadIdx.x;
    if (c < nchunks) {
        const Chunk va = load_chunk_as<kStream>(a + c);
        const Chunk vb = load_chunk_as<kStream>(b + c);
        store_chunk_as<kStream>(out + c, apply2<kOp>(va, vb));
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
        const size_t blocks = nchunks ? (nchunks + kEwBlock - 1) / kEwBlock : 1;
        if (use_streaming(3u * n * 2u))
            binary_chunks<kOp, true><<<dim3((unsigned)blocks), kEwBlock, 0, st>>>(
                static_cast<const Chunk*>(a), static_cast<const Chunk*>(b),
                static_cast<Chunk*>(out), nchunks, tail);
        else
            binary_chunks<kOp, false><<<dim3((unsigned)blocks), kEwBlock, 0, st>>>(
                static_cast<const Chunk*>(a), static_cast<const Chunk*>(b),
                static_cast<Chunk*>(out), nchunks, tail);
    } else {
        const size_t blocks = (n + kBlock - 1) / kBlock;
        binary_halves<kOp><<<dim3((unsigned)blocks), kBlock, 0, st>>>(
            static_cast<const h16*>(a), static_cast<const h16*>(b), static_cast<h16*>(out), n);
    }
    return launch_status();
}

// gate and up are the two halves of each [2*inter] row; flat over the output.
__global__ __launch_bounds__(kEwBlock) void swiglu_fused_chunks(const Chunk* gate_up, Chunk* out,
                                                                size_t total_chunks,
                                                                int inter_chunks) {
    const size_t c = (size_t)blockIdx.x * kEwBlock + threadIdx.x;
    if (c < total_chunks) {
        const size_t row = c / (size_t)inter_chunks, col = c - row * (size_t)inter_chunks;
        const Chunk* g = gate_up + row * 2u * (size_t)inter_chunks + col;
        store_chunk(out + c, apply2<kSwiglu>(load_chunk(g), load_chunk(g + inter_chunks)));
    }
}

__global__ __launch_bounds__(kBlock) void swiglu_fused_halves(const h16* gate_up, h16* out,
                                                              size_t total, int inter) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < total) {
        const size_t row = i / (size_t)inter, col = i - row * (size_t)inter;
        const h16* g = gate_up + row * 2u * (size_t)inter + col;
        out[i] = apply2<kSwiglu>(g[0], g[inter]);
    }
}

// out[m, :] += bias[:]. Chunked form: a row is n_chunks chunks, the bias chunk
// index is the chunk's column, found with one 64-bit modulo per chunk.
__global__ __launch_bounds__(kEwBlock) void bias_add_chunks(Chunk* out, const Chunk* __restrict__ bias,
                                                            size_t total_chunks, int row_chunks) {
    const size_t c = (size_t)blockIdx.x * kEwBlock + threadIdx.x;
    if (c < total_chunks) {
        const Chunk v = load_chunk(out + c);
        const Chunk bv = load_chunk(bias + (c % (size_t)row_chunks));
        store_chunk(out + c, apply2<kResidual>(v, bv));
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
    const size_t total = (size_t)rows * (size_t)inter;
    if (inter % 8 == 0 && vv::aligned16(gate_up) && vv::aligned16(output)) {
        const size_t chunks = total / 8;
        vv::swiglu_fused_chunks<<<dim3((unsigned)((chunks + vv::kEwBlock - 1) / vv::kEwBlock)),
                                  vv::kEwBlock, 0, st>>>(
            static_cast<const vv::Chunk*>(gate_up), static_cast<vv::Chunk*>(output), chunks,
            inter / 8);
    } else {
        vv::swiglu_fused_halves<<<dim3((unsigned)((total + vv::kBlock - 1) / vv::kBlock)),
                                  vv::kBlock, 0, st>>>(
            static_cast<const vv::h16*>(gate_up), static_cast<vv::h16*>(output), total, inter);
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
        const size_t blocks = (chunks + vv::kEwBlock - 1) / vv::kEwBlock;
        vv::bias_add_chunks<<<dim3((unsigned)blocks), vv::kEwBlock, 0, st>>>(
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
